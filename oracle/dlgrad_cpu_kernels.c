/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Plain-C restatement of the kernels dlgrad generates for its CPU device
 * (/root/reference/dlgrad/codegen/cpu_kernel.py).  Same loop nests, same loop
 * order, same int/float conversions, same zero-initialisation expectations; each
 * function cites the generator lines it follows.  Built with the reference's own
 * flags (dlgrad/runtime/cpu.py:30-41: -O3 -march=native -ffast-math, clang if
 * present else gcc, -lm -lmvec).  It is the checker the HIP kernels are compared
 * with and the single-threaded CPU baseline the benchmark reports; only tests/,
 * the smoke check and the benchmark's cpu_baseline leg may load it.
 *
 * The reference emits one function per rank ("add_3d", "where_2d", ...).  The
 * macros below stamp out the same per-rank functions so the compiler sees the
 * same loop structure; the *_nd entry points only select by rank.
 *
 * How each function is pinned (tests/test_oracle.py) -- never by re-typing the
 * formula, always by an independent statement of the result:
 *   arithmetic / comparisons / where / masked_fill / clamp / cmp  numpy broadcasting on fp32 (bit-exact for + - * selects)
 *   neg exp log pow sqrt rsqrt     numpy float64 then rounded to fp32
 *   reduce / reduce_axis           numpy float64 reductions; max bit-exact
 *   argmax                         numpy argmax, planted ties resolve to the first index
 *   permute                        np.transpose(...).copy(), bit-exact
 *   matmul 2/3/4-D                 np.matmul in float64, brute force on tiny cases, broadcast batches
 *   embedding / embedding_backward table[idx] bit-exact; np.add.at in float64
 *   ce_forward / ce_backward       fancy indexing closed forms
 *   full / arange / init_with_scalar  closed forms incl. the int truncation
 * uniform (cpu_kernel.py:774-874) reseeds itself from /dev/random on every call
 * and cannot be pinned value-for-value: parity unpinned; only its range and
 * moments are tested.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- arithmetic: cpu_kernel.py:12-66 ---------------------------------------
 * out[ptr++] = x[sum i_d*xs_d] OP y[sum i_d*ys_d], loops over the out shape,
 * outermost dim first; comparisons yield 0/1 as float.                        */
#define ARITH_ND(NAME, EXPR)                                                                  \
    static void NAME##_0d(const float *x, const float *y, float *out, const int *shape,      \
                          const int *xs, const int *ys) {                                     \
        (void)shape; (void)xs; (void)ys;                                                      \
        int ptr = 0; int x_idx = 0; int y_idx = 0;                                            \
        float a = x[x_idx], b = y[y_idx]; out[ptr++] = EXPR;                                  \
    }                                                                                         \
    static void NAME##_1d(const float *x, const float *y, float *out, const int *shape,      \
                          const int *xs, const int *ys) {                                     \
        int ptr = 0;                                                                          \
        for (int i0 = 0; i0 < shape[0]; i0++) {                                               \
            int x_idx = i0 * xs[0]; int y_idx = i0 * ys[0];                                   \
            float a = x[x_idx], b = y[y_idx]; out[ptr++] = EXPR;                              \
        }                                                                                     \
    }                                                                                         \
    static void NAME##_2d(const float *x, const float *y, float *out, const int *shape,      \
                          const int *xs, const int *ys) {                                     \
        int ptr = 0;                                                                          \
        for (int i0 = 0; i0 < shape[0]; i0++)                                                 \
            for (int i1 = 0; i1 < shape[1]; i1++) {                                           \
                int x_idx = i0 * xs[0] + i1 * xs[1]; int y_idx = i0 * ys[0] + i1 * ys[1];     \
                float a = x[x_idx], b = y[y_idx]; out[ptr++] = EXPR;                          \
            }                                                                                 \
    }                                                                                         \
    static void NAME##_3d(const float *x, const float *y, float *out, const int *shape,      \
                          const int *xs, const int *ys) {                                     \
        int ptr = 0;                                                                          \
        for (int i0 = 0; i0 < shape[0]; i0++)                                                 \
            for (int i1 = 0; i1 < shape[1]; i1++)                                             \
                for (int i2 = 0; i2 < shape[2]; i2++) {                                       \
                    int x_idx = i0 * xs[0] + i1 * xs[1] + i2 * xs[2];                         \
                    int y_idx = i0 * ys[0] + i1 * ys[1] + i2 * ys[2];                         \
                    float a = x[x_idx], b = y[y_idx]; out[ptr++] = EXPR;                      \
                }                                                                             \
    }                                                                                         \
    static void NAME##_4d(const float *x, const float *y, float *out, const int *shape,      \
                          const int *xs, const int *ys) {                                     \
        int ptr = 0;                                                                          \
        for (int i0 = 0; i0 < shape[0]; i0++)                                                 \
            for (int i1 = 0; i1 < shape[1]; i1++)                                             \
                for (int i2 = 0; i2 < shape[2]; i2++)                                         \
                    for (int i3 = 0; i3 < shape[3]; i3++) {                                   \
                        int x_idx = i0 * xs[0] + i1 * xs[1] + i2 * xs[2] + i3 * xs[3];        \
                        int y_idx = i0 * ys[0] + i1 * ys[1] + i2 * ys[2] + i3 * ys[3];        \
                        float a = x[x_idx], b = y[y_idx]; out[ptr++] = EXPR;                  \
                    }                                                                         \
    }                                                                                         \
    void ref_##NAME(const float *x, const float *y, float *out, int ndim, const int *shape,  \
                    const int *xs, const int *ys) {                                           \
        switch (ndim) {                                                                       \
            case 0: NAME##_0d(x, y, out, shape, xs, ys); break;                               \
            case 1: NAME##_1d(x, y, out, shape, xs, ys); break;                               \
            case 2: NAME##_2d(x, y, out, shape, xs, ys); break;                               \
            case 3: NAME##_3d(x, y, out, shape, xs, ys); break;                               \
            default: NAME##_4d(x, y, out, shape, xs, ys); break;                              \
        }                                                                                     \
    }

ARITH_ND(add, a + b)
ARITH_ND(sub, a - b)
ARITH_ND(mul, a * b)
ARITH_ND(div, a / b)
ARITH_ND(eq, a == b)
ARITH_ND(lt, a < b)
ARITH_ND(gt, a > b)
ARITH_ND(gte, a >= b)

/* ---- cmp_2d("<="): cpu_kernel.py:653-668 ------------------------------------- */
void ref_cmp_le(const float *x, const float *y, float *out, const int *out_shape, const int *xs,
                const int *ys, const int *os) {
    for (int i = 0; i < out_shape[0]; i++)
        for (int j = 0; j < out_shape[1]; j++) {
            int x_idx = i * xs[0] + j * xs[1];
            int y_idx = i * ys[0] + j * ys[1];
            out[i * os[0] + j * os[1]] = x[x_idx] <= y[y_idx] ? 1.0 : 0.0;
        }
}

/* ---- flat unary kernels: cpu_kernel.py:246-319 --------------------------------
 * exp and log are the double-precision libm calls on a promoted float; pow takes
 * an int exponent (the caller truncates, cpu.py:500).                             */
void ref_neg(const float *x, float *out, int n) { for (int i = 0; i < n; i++) out[i] = -1 * x[i]; }
void ref_exp(const float *x, float *out, int n) { for (int i = 0; i < n; i++) out[i] = exp(x[i]); }
void ref_log(const float *x, float *out, int n) { for (int i = 0; i < n; i++) out[i] = log(x[i]); }
void ref_pow(const float *x, float *out, int n, int val) { for (int i = 0; i < n; i++) out[i] = powf(x[i], val); }
void ref_sqrt(const float *x, float *out, int n) { for (int i = 0; i < n; i++) out[i] = sqrtf(x[i]); }
void ref_rsqrt(const float *x, float *out, int n) { for (int i = 0; i < n; i++) out[i] = 1.0 / sqrtf(x[i]); }

/* relu: cpu_kernel.py:520-533 (registered, never dispatched by Buffer) */
void ref_relu(const float *arr, float *out, int n) {
    for (int i = 0; i < n; i++) out[i] = (arr[i] <= 0) ? 0.0f : arr[i];
}

/* clamp: cpu_kernel.py:321-349; absent bounds are skipped */
void ref_clamp(const float *x, float *out, int numel, int has_min, float min_val, int has_max,
               float max_val) {
    if (has_min && has_max) {
        for (int i = 0; i < numel; i++) { float v = x[i]; if (v < min_val) v = min_val; if (v > max_val) v = max_val; out[i] = v; }
    } else if (has_min) {
        for (int i = 0; i < numel; i++) { float v = x[i]; if (v < min_val) v = min_val; out[i] = v; }
    } else if (has_max) {
        for (int i = 0; i < numel; i++) { float v = x[i]; if (v > max_val) v = max_val; out[i] = v; }
    } else {
        for (int i = 0; i < numel; i++) out[i] = x[i];
    }
}

/* ---- full reductions: cpu_kernel.py:150-177 ------------------------------------- */
void ref_reduce_sum(const float *x, float *out, int numel) {
    float val = 0;
    for (int i = 0; i < numel; i++) val += x[i];
    out[0] = val;
}
void ref_reduce_mean(const float *x, float *out, int numel) {
    float val = 0;
    for (int i = 0; i < numel; i++) val += x[i];
    out[0] = val / numel;
}
void ref_reduce_max(const float *x, float *out, int numel) {
    float val = -FLT_MAX;
    for (int i = 0; i < numel; i++) if (x[i] > val) val = x[i];
    out[0] = val;
}

/* ---- reductions along one axis: cpu_kernel.py:68-148 -------------------------------
 * Outer loops over the kept dims in order, inner sequential loop over the reduced
 * dim with the input strides; out index uses out_stride[k] for the k-th kept dim.
 * Written once over a rank padded to 4 on the left (extent 1, stride 0), which
 * visits the same elements in the same order as the per-rank functions.           */
#define AXIS_REDUCE(NAME, INIT, UPDATE, FINAL)                                                   \
    void ref_reduce_##NAME##_axis(const float *x, float *out, int ndim, int reduce_dim,          \
                                  const int *shape, const int *x_stride, const int *out_stride) { \
        int sh[4] = {1, 1, 1, 1}, xs[4] = {0, 0, 0, 0}, os[4] = {0, 0, 0, 0};                    \
        int pad = 4 - ndim, k = 0;                                                               \
        for (int d = 0; d < ndim; d++) {                                                         \
            sh[pad + d] = shape[d]; xs[pad + d] = x_stride[d];                                   \
            if (d != reduce_dim) os[pad + d] = out_stride[k++];                                  \
        }                                                                                        \
        int rd = pad + reduce_dim, n = sh[rd], rs = xs[rd];                                      \
        int o[4];                                                                                \
        for (int d = 0; d < 4; d++) o[d] = (d == rd) ? 1 : sh[d];                                \
        for (int i0 = 0; i0 < o[0]; i0++)                                                        \
            for (int i1 = 0; i1 < o[1]; i1++)                                                    \
                for (int i2 = 0; i2 < o[2]; i2++)                                                \
                    for (int i3 = 0; i3 < o[3]; i3++) {                                          \
                        int base = i0 * xs[0] + i1 * xs[1] + i2 * xs[2] + i3 * xs[3];            \
                        INIT;                                                                    \
                        for (int r = 0; r < n; r++) { float v = x[base + r * rs]; UPDATE; }      \
                        out[i0 * os[0] + i1 * os[1] + i2 * os[2] + i3 * os[3]] = FINAL;          \
                    }                                                                            \
    }
AXIS_REDUCE(sum, float val = 0, val += v, val)
AXIS_REDUCE(mean, float val = 0, val += v, val / n)
AXIS_REDUCE(max, float val = -FLT_MAX, if (v > val) val = v, val)

/* ---- argmax: cpu_kernel.py:459-517 --------------------------------------------------
 * strict '>' so the first maximum wins; starts at -FLT_MAX with index 0; the index
 * is written as a float.                                                            */
void ref_argmax_axis(const float *x, float *out, int ndim, int reduce_dim, const int *shape,
                     const int *x_stride, const int *out_stride) {
    int sh[4] = {1, 1, 1, 1}, xs[4] = {0, 0, 0, 0}, os[4] = {0, 0, 0, 0};
    int pad = 4 - ndim, k = 0;
    for (int d = 0; d < ndim; d++) {
        sh[pad + d] = shape[d]; xs[pad + d] = x_stride[d];
        if (d != reduce_dim) os[pad + d] = out_stride[k++];
    }
    int rd = pad + reduce_dim, n = sh[rd], rs = xs[rd];
    int o[4];
    for (int d = 0; d < 4; d++) o[d] = (d == rd) ? 1 : sh[d];
    for (int i0 = 0; i0 < o[0]; i0++)
        for (int i1 = 0; i1 < o[1]; i1++)
            for (int i2 = 0; i2 < o[2]; i2++)
                for (int i3 = 0; i3 < o[3]; i3++) {
                    int base = i0 * xs[0] + i1 * xs[1] + i2 * xs[2] + i3 * xs[3];
                    float max_val = -3.402823466e+38F;
                    int best_idx = 0;
                    for (int r = 0; r < n; r++) {
                        float v = x[base + r * rs];
                        if (v > max_val) { max_val = v; best_idx = r; }
                    }
                    out[i0 * os[0] + i1 * os[1] + i2 * os[2] + i3 * os[3]] = (float)best_idx;
                }
}

/* ---- permute: cpu_kernel.py:179-215 ----------------------------------------------------
 * loops over the OUT shape; in_strides are the input strides reordered by `order`. */
void ref_permute(const float *x, float *out, int ndim, const int *shape, const int *in_strides,
                 const int *out_strides) {
    int sh[4] = {1, 1, 1, 1}, is[4] = {0, 0, 0, 0}, os[4] = {0, 0, 0, 0};
    int pad = 4 - ndim;
    for (int d = 0; d < ndim; d++) { sh[pad + d] = shape[d]; is[pad + d] = in_strides[d]; os[pad + d] = out_strides[d]; }
    for (int i0 = 0; i0 < sh[0]; i0++)
        for (int i1 = 0; i1 < sh[1]; i1++)
            for (int i2 = 0; i2 < sh[2]; i2++)
                for (int i3 = 0; i3 < sh[3]; i3++) {
                    int in_idx = i0 * is[0] + i1 * is[1] + i2 * is[2] + i3 * is[3];
                    int out_idx = i0 * os[0] + i1 * os[1] + i2 * os[2] + i3 * os[3];
                    out[out_idx] = x[in_idx];
                }
}

/* ---- where: cpu_kernel.py:535-587; masked_fill: cpu_kernel.py:603-650 -------------------- */
void ref_where(const float *cond, const float *x, const float *y, float *out, int ndim,
               const int *shape, const int *c_stride, const int *x_stride, const int *y_stride,
               const int *out_stride) {
    int sh[4] = {1, 1, 1, 1}, cs[4] = {0}, xs[4] = {0}, ys[4] = {0}, os[4] = {0};
    int pad = 4 - ndim;
    for (int d = 0; d < ndim; d++) {
        sh[pad + d] = shape[d]; cs[pad + d] = c_stride[d]; xs[pad + d] = x_stride[d];
        ys[pad + d] = y_stride[d]; os[pad + d] = out_stride[d];
    }
    for (int i0 = 0; i0 < sh[0]; i0++)
        for (int i1 = 0; i1 < sh[1]; i1++)
            for (int i2 = 0; i2 < sh[2]; i2++)
                for (int i3 = 0; i3 < sh[3]; i3++) {
                    int c_idx = i0 * cs[0] + i1 * cs[1] + i2 * cs[2] + i3 * cs[3];
                    int x_idx = i0 * xs[0] + i1 * xs[1] + i2 * xs[2] + i3 * xs[3];
                    int y_idx = i0 * ys[0] + i1 * ys[1] + i2 * ys[2] + i3 * ys[3];
                    int out_idx = i0 * os[0] + i1 * os[1] + i2 * os[2] + i3 * os[3];
                    out[out_idx] = (cond[c_idx] > 0) ? x[x_idx] : y[y_idx];
                }
}

void ref_masked_fill(const float *x, const float *mask, float *out, int ndim, const int *shape,
                     const int *x_stride, const int *mask_stride, const int *out_stride,
                     float fill_value) {
    int sh[4] = {1, 1, 1, 1}, xs[4] = {0}, ms[4] = {0}, os[4] = {0};
    int pad = 4 - ndim;
    for (int d = 0; d < ndim; d++) {
        sh[pad + d] = shape[d]; xs[pad + d] = x_stride[d]; ms[pad + d] = mask_stride[d];
        os[pad + d] = out_stride[d];
    }
    for (int i0 = 0; i0 < sh[0]; i0++)
        for (int i1 = 0; i1 < sh[1]; i1++)
            for (int i2 = 0; i2 < sh[2]; i2++)
                for (int i3 = 0; i3 < sh[3]; i3++) {
                    int x_idx = i0 * xs[0] + i1 * xs[1] + i2 * xs[2] + i3 * xs[3];
                    int mask_idx = i0 * ms[0] + i1 * ms[1] + i2 * ms[2] + i3 * ms[3];
                    int out_idx = i0 * os[0] + i1 * os[1] + i2 * os[2] + i3 * os[3];
                    out[out_idx] = (mask[mask_idx] > 0) ? fill_value : x[x_idx];
                }
}

/* ---- matmul: cpu_kernel.py:351-428 --------------------------------------------------------
 * out must arrive zeroed (cpu.py:517,549,579); i-k-j order, one FMA chain per output
 * in increasing k.                                                                     */
void ref_matmul_2d(const float *x, const float *y, float *out, const int *x_shape,
                   const int *x_stride, const int *y_shape, const int *y_stride) {
    for (int i = 0; i < x_shape[0]; i++)
        for (int k = 0; k < x_shape[1]; k++) {
            float a = x[i * x_stride[0] + k * x_stride[1]];
            for (int j = 0; j < y_shape[1]; j++)
                out[i * y_shape[1] + j] += a * y[k * y_stride[0] + j * y_stride[1]];
        }
}

void ref_matmul_3d(const float *x, const float *y, float *out, int B, int M, int K, int N,
                   const int *sx, const int *sy, const int *so) {
    for (int b = 0; b < B; b++)
        for (int i = 0; i < M; i++)
            for (int k = 0; k < K; k++) {
                float a = x[b * sx[0] + i * sx[1] + k * sx[2]];
                for (int j = 0; j < N; j++) {
                    int y_idx = b * sy[0] + k * sy[1] + j * sy[2];
                    int out_idx = b * so[0] + i * so[1] + j * so[2];
                    out[out_idx] += a * y[y_idx];
                }
            }
}

void ref_matmul_4d(const float *x, const float *y, float *out, const int *dims,
                   const int *x_stride, const int *y_stride, const int *out_stride) {
    int B = dims[0], C = dims[1], M = dims[2], K = dims[3], N = dims[4];
    for (int b = 0; b < B; ++b)
        for (int c = 0; c < C; ++c) {
            const float *A_ptr = x + (b * x_stride[0]) + (c * x_stride[1]);
            const float *B_ptr = y + (b * y_stride[0]) + (c * y_stride[1]);
            float *out_ptr = out + (b * out_stride[0]) + (c * out_stride[1]);
            for (int h = 0; h < M; ++h) {
                const float *A_row = A_ptr + (h * x_stride[2]);
                float *out_row = out_ptr + (h * out_stride[2]);
                for (int k = 0; k < K; ++k) {
                    float a_val = A_row[k * x_stride[3]];
                    const float *B_row_k = B_ptr + (k * y_stride[2]);
                    for (int w = 0; w < N; ++w)
                        out_row[w * out_stride[3]] += a_val * B_row_k[w * y_stride[3]];
                }
            }
        }
}

/* ---- embedding: cpu_kernel.py:217-243 --------------------------------------------------------
 * forward: row index = (int)(idx[i]*W) computed in float then truncated.
 * backward as the reference has it: the flat index idx[i]*W + j is evaluated in
 * FLOAT (wrong above 2^24), out must arrive zeroed, rows accumulate in index order.
 * ref_embedding_backward_int is the same loop with the index formed in integers,
 * i.e. what the float expression means wherever it is exact.                          */
void ref_embedding(const float *x, const float *idx, float *out, int idx_numel, int x_width) {
    for (int i = 0; i < idx_numel; i++) {
        int x_idx = idx[i] * x_width;
        memcpy(&out[i * x_width], &x[x_idx], x_width * sizeof(float));
    }
}
void ref_embedding_backward(float *out, const float *upstream_grad, const float *idx,
                            int idx_numel, int x_width) {
    for (int i = 0; i < idx_numel; i++)
        for (int j = 0; j < x_width; j++) {
            int x_idx = idx[i] * x_width + j;
            out[x_idx] += upstream_grad[i * x_width + j];
        }
}
void ref_embedding_backward_int(float *out, const float *upstream_grad, const float *idx,
                                int idx_numel, int x_width) {
    for (int i = 0; i < idx_numel; i++) {
        int row = (int)idx[i];
        for (int j = 0; j < x_width; j++)
            out[row * x_width + j] += upstream_grad[i * x_width + j];
    }
}

/* ---- cross-entropy helpers: cpu_kernel.py:430-457 ------------------------------------------------ */
void ref_ce_forward(const float *x, const float *target, float *out, int n_rows, const int *x_stride) {
    for (int i = 0; i < n_rows; i++) out[i] = x[(int)target[i] + (x_stride[0] * i)];
}
void ref_ce_backward(float *x, const float *target, const int *x_shape, const int *x_stride) {
    int rows = x_shape[0];
    for (int i = 0; i < rows; i++) x[(int)target[i] + (x_stride[0] * i)] -= 1;
}

/* ---- fills: cpu_kernel.py:707-770 -- note the int arguments ---------------------------------------- */
void ref_init_with_scalar(float *out, int numel, int scalar) { for (int i = 0; i < numel; i++) out[i] = scalar; }
void ref_arange(float *out, int x_numel) { for (int i = 0; i < x_numel; i++) out[i] = i; }
void ref_full(float *out, int x_numel, int fill_value) { for (int i = 0; i < x_numel; i++) out[i] = fill_value; }
void ref_full_f(float *out, int x_numel, float fill_value) { for (int i = 0; i < x_numel; i++) out[i] = fill_value; }

/* ---- uniform: cpu_kernel.py:774-874 --------------------------------------------------------------------
 * PCG32 (O'Neill, pcg_basic): state*6364136223846793005+inc, XSH-RR output,
 * f = (float)ldexp(u32, -32), low + (high-low)*f.  The reference seeds from
 * /dev/random on every call; here the seed is an argument so runs repeat.          */
typedef struct { uint64_t state, inc; } ref_pcg32_t;
static uint32_t ref_pcg32_next(ref_pcg32_t *r) {
    uint64_t old = r->state;
    r->state = old * 6364136223846793005ULL + r->inc;
    uint32_t xorshifted = (uint32_t)(((old >> 18u) ^ old) >> 27u);
    uint32_t rot = (uint32_t)(old >> 59u);
    return (xorshifted >> rot) | (xorshifted << ((-rot) & 31));
}
void ref_uniform(float *out, int numel, float low, float high, uint64_t initstate, uint64_t initseq) {
    ref_pcg32_t r = {0u, (initseq << 1u) | 1u};
    ref_pcg32_next(&r);
    r.state += initstate;
    ref_pcg32_next(&r);
    for (int i = 0; i < numel; i++) {
        float f = (float)ldexp(ref_pcg32_next(&r), -32);
        out[i] = low + (high - low) * f;
    }
}
/* raw generator outputs, so the PCG32 restatement can be checked against the
 * published pcg32 demo vector (seed 42, sequence 54). */
void ref_pcg32_raw(uint32_t *out, int n, uint64_t initstate, uint64_t initseq) {
    ref_pcg32_t r = {0u, (initseq << 1u) | 1u};
    ref_pcg32_next(&r);
    r.state += initstate;
    ref_pcg32_next(&r);
    for (int i = 0; i < n; i++) out[i] = ref_pcg32_next(&r);
}
