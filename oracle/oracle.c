/*
 * CPU oracle: a plain-C restatement of the reference's algorithms for the hot path
 * (ZhengChenCS/CompressGNN; paths below are relative to its root).
 *
 * TEST INFRASTRUCTURE ONLY.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load this library; the product never does.
 *
 * How each function is pinned (what would catch a dropped term, wrong index, wrong
 * sign or transposed operand) is listed in oracle/README.md and checked by
 * tests/test_oracle_*.py:
 *   - spmm_*           : outputs of the reference's own compiled spmm_func (golden
 *                        vectors and, where built, oracle/_ref), dense float64 products
 *   - lsh_*            : the torch restatement of the reference's own test
 *                        (tests/test_transformation.py:16-20), golden (index, active) of
 *                        the compiled cluster_forward on inputs whose projections are
 *                        exactly representable, known answers count == [0, 513]
 *   - the sampler (oracle_sample.c) : the compiled reference's own outputs, its draws replayed
 *                        from torch's CPU generator; its counter-based generator is this
 *                        build's definition and "parity unpinned" (see that file's header)
 *   - cluster_mean_*, reconstruct_* : index_add / index_select closed forms of
 *                        layer/CompressgnnCluster.py:16-25 and
 *                        layer/CompressgnnReconstruct.py:39-42, float64 finite differences
 *
 * Build: make -C oracle  (gcc -O3 -fopenmp -ffp-contract=off, no -march: products
 * and sums are rounded separately, as in the reference build src/runtime/setup.py:30).
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---- SpMM, "rowbalance" schedule: src/runtime/csrc/sparse/cpu/spmm_cpu.cpp:42-70 ----
 * out[r,:] += vals, vals = ((0 + m0*v0) + m1*v1) + ... over the entries of row r in
 * ascending order; out must hold the values to accumulate onto (zeros for a fresh
 * result, spmm_cpu.cpp:24-28).  threads <= 1 runs serially. */
#define DEFINE_SPMM(NAME, T)                                                              \
    void NAME(int64_t rows, const int64_t *vlist, const int64_t *elist, const T *value,   \
              const T *mat, int64_t F, T *out, int threads) {                             \
        if (rows <= 0 || F <= 0) return;                                                  \
        if (threads < 1) threads = 1;                                                     \
        _Pragma("omp parallel num_threads(threads)")                                      \
        {                                                                                 \
            T *vals = (T *)malloc(sizeof(T) * (size_t)F);                                 \
            _Pragma("omp for schedule(static)")                                           \
            for (int64_t r = 0; r < rows; ++r) {                                          \
                for (int64_t k = 0; k < F; ++k) vals[k] = 0;                              \
                for (int64_t e = vlist[r]; e < vlist[r + 1]; ++e) {                       \
                    const T v = value[e];                                                 \
                    const T *m = mat + elist[e] * F;                                      \
                    for (int64_t k = 0; k < F; ++k) vals[k] += m[k] * v;                  \
                }                                                                         \
                T *o = out + r * F;                                                       \
                for (int64_t k = 0; k < F; ++k) o[k] += vals[k];                          \
            }                                                                             \
            free(vals);                                                                   \
        }                                                                                 \
    }
DEFINE_SPMM(oracle_spmm_f32, float)
DEFINE_SPMM(oracle_spmm_f64, double)

/* ---- LSH assignment: src/runtime/csrc/cluster/cpu/cluster_cpu.cpp:27-70 -------------
 * The reference projects with torch mm, whose summation order is the BLAS library's;
 * this build fixes the order instead: h_j = fma(x_k, w_kj, h_j), k ascending, h_j = 0
 * at the start.  Bits are packed most significant first with a strict "> 0" test
 * (cluster_cpu.cpp:47-54); dense ids are the inclusive prefix of bucket occupancy,
 * hence 1-based (cluster_cpu.cpp:58-67).  raw_code may be NULL. */
#define DEFINE_LSH(NAME, T, FMA)                                                          \
    void NAME(int64_t N, int64_t F, int H, const T *X, const T *W, int32_t *index,        \
              int32_t *active, int32_t *raw_code) {                                       \
        const int64_t buckets = (int64_t)1 << H;                                          \
        unsigned char *flag = (unsigned char *)calloc((size_t)buckets, 1);                \
        int32_t *dense = (int32_t *)malloc(sizeof(int32_t) * (size_t)buckets);            \
        T h[32];                                                                          \
        for (int64_t i = 0; i < N; ++i) {                                                 \
            for (int j = 0; j < H; ++j) h[j] = 0;                                         \
            for (int64_t k = 0; k < F; ++k) {                                             \
                const T x = X[i * F + k];                                                 \
                for (int j = 0; j < H; ++j) h[j] = FMA(x, W[k * H + j], h[j]);            \
            }                                                                             \
            int32_t id = 0;                                                               \
            for (int j = 0; j < H; ++j) id = (id << 1) | (h[j] > 0 ? 1 : 0);              \
            index[i] = id;                                                                \
            if (raw_code) raw_code[i] = id;                                               \
            flag[id] = 1;                                                                 \
        }                                                                                 \
        int32_t run = 0;                                                                  \
        for (int64_t b = 0; b < buckets; ++b) {                                           \
            run += flag[b];                                                               \
            dense[b] = run;                                                               \
        }                                                                                 \
        *active = run;                                                                    \
        for (int64_t i = 0; i < N; ++i) index[i] = dense[index[i]];                       \
        free(flag);                                                                       \
        free(dense);                                                                      \
    }
DEFINE_LSH(oracle_lsh_f32, float, fmaf)
DEFINE_LSH(oracle_lsh_f64, double, fma)

/* ---- mean representatives: layer/CompressgnnCluster.py:16-19 (scatter_mean) and
 * src/runtime/csrc/cluster/cuda/cluster_kernel.cu:60-75 -------------------------------
 * reps[g,:] = (sum of x[i,:] over i with index[i] == g, i ascending) / max(count[g],1);
 * reps has `groups` rows. */
#define DEFINE_MEAN(NAME, T)                                                              \
    void NAME(int64_t N, int64_t F, int64_t groups, const T *X, const int64_t *index,     \
              const int32_t *count, T *reps) {                                            \
        memset(reps, 0, sizeof(T) * (size_t)(groups * F));                                \
        for (int64_t i = 0; i < N; ++i) {                                                 \
            T *r = reps + index[i] * F;                                                   \
            const T *x = X + i * F;                                                       \
            for (int64_t k = 0; k < F; ++k) r[k] += x[k];                                 \
        }                                                                                 \
        for (int64_t g = 0; g < groups; ++g) {                                            \
            const T d = (T)(count[g] > 1 ? count[g] : 1);                                 \
            for (int64_t k = 0; k < F; ++k) reps[g * F + k] /= d;                         \
        }                                                                                 \
    }
DEFINE_MEAN(oracle_cluster_mean_f32, float)
DEFINE_MEAN(oracle_cluster_mean_f64, double)

/* ---- mean backward: layer/CompressgnnCluster.py:22-25, cluster_kernel.cu:76-85 ------
 * dx[i,:] = grad[index[i],:] / max(count[index[i]],1) */
#define DEFINE_MEAN_BWD(NAME, T)                                                          \
    void NAME(int64_t N, int64_t F, const T *grad, const int64_t *index,                  \
              const int32_t *count, T *dx, int threads) {                                 \
        if (threads < 1) threads = 1;                                                     \
        _Pragma("omp parallel for schedule(static) num_threads(threads)")                 \
        for (int64_t i = 0; i < N; ++i) {                                                 \
            const int64_t g = index[i];                                                   \
            const T d = (T)(count[g] > 1 ? count[g] : 1);                                 \
            for (int64_t k = 0; k < F; ++k) dx[i * F + k] = grad[g * F + k] / d;          \
        }                                                                                 \
    }
DEFINE_MEAN_BWD(oracle_cluster_mean_backward_f32, float)
DEFINE_MEAN_BWD(oracle_cluster_mean_backward_f64, double)

/* ---- reconstruct: layer/CompressgnnReconstruct.py:39-42, cluster_kernel.cu:86-97 -----
 * out[i,:] = act(reps[index[i],:] + bias), act(v) = (relu && v < 0) ? 0 : v */
#define DEFINE_RECON(NAME, T)                                                             \
    void NAME(int64_t N, int64_t F, const T *reps, const int64_t *index, const T *bias,   \
              int relu, T *out, int threads) {                                            \
        if (threads < 1) threads = 1;                                                     \
        _Pragma("omp parallel for schedule(static) num_threads(threads)")                 \
        for (int64_t i = 0; i < N; ++i) {                                                 \
            const T *r = reps + index[i] * F;                                             \
            for (int64_t k = 0; k < F; ++k) {                                             \
                T v = r[k];                                                               \
                if (bias) v += bias[k];                                                   \
                out[i * F + k] = (relu && v < 0) ? (T)0 : v;                              \
            }                                                                             \
        }                                                                                 \
    }
DEFINE_RECON(oracle_reconstruct_f32, float)
DEFINE_RECON(oracle_reconstruct_f64, double)

/* ---- reconstruct backward: cluster_kernel.cu:98-108 ---------------------------------
 * reps_grad[g,:] = sum over i with index[i] == g (ascending) of
 *                  ((relu && output[i,:] <= 0) ? 0 : grad[i,:]) */
#define DEFINE_RECON_BWD(NAME, T)                                                         \
    void NAME(int64_t N, int64_t F, int64_t groups, const T *grad, const T *output,       \
              const int64_t *index, int relu, T *reps_grad) {                             \
        memset(reps_grad, 0, sizeof(T) * (size_t)(groups * F));                           \
        for (int64_t i = 0; i < N; ++i) {                                                 \
            T *r = reps_grad + index[i] * F;                                              \
            for (int64_t k = 0; k < F; ++k) {                                             \
                const T g = (relu && output[i * F + k] <= 0) ? (T)0 : grad[i * F + k];    \
                r[k] += g;                                                                \
            }                                                                             \
        }                                                                                 \
    }
DEFINE_RECON_BWD(oracle_reconstruct_backward_f32, float)
DEFINE_RECON_BWD(oracle_reconstruct_backward_f64, double)

int oracle_max_threads(void) { return omp_get_max_threads(); }
