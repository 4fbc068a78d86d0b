/*
 * Brute-force restatement of the FlashMoE forward stages in plain C.  TEST INFRASTRUCTURE ONLY.
 *
 * Purpose: an implementation that shares no code, library routine or algorithmic shortcut with
 * either the torch oracle (oracle/flashmoe_oracle.py) or the HIP kernels, so that the oracle can
 * be pinned against it on small and medium inputs.  Everything is explicit loops; the floating
 * point stages accumulate in double.
 *
 * What each function restates (reference = flash-algo/flash-moe):
 *   bf_router_topk   the definition in docs/flash_router.md:5-11 and the exhaustive selection of
 *                    flash_moe/ops/triton/flash_router.py:33-63: all nk*nk sums lp[0,t,i]+lp[1,t,j]
 *                    (added in float, as the fp32 reference does), K largest, ties to the lowest
 *                    flat index i*nk+j (tl.argmax's rule, flash_router.py:58).
 *   bf_prologue      flash_moe/modules/flash_moe.py:147-156: batch statistics (biased variance,
 *                    eps 1e-5) or given running statistics, normalise, x Wr^T, log-softmax per half.
 *   bf_expert        flash_moe/modules/flash_moe.py:178-186 / docs/flash_expert.md:5-9.
 *   bf_mlp           flash_moe/modules/flash_moe.py:187-189 / tests/test_mlp.py:9-19.
 *
 * Build: gcc -O2 -shared -fPIC -o _build/libbruteforce.so bruteforce.c -lm   (see oracle/Makefile)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct { float score; int64_t flat; } bf_pair;

static int bf_pair_cmp(const void* pa, const void* pb) {
    const bf_pair* a = (const bf_pair*)pa;
    const bf_pair* b = (const bf_pair*)pb;
    if (a->score > b->score) return -1;
    if (a->score < b->score) return 1;
    if (a->flat < b->flat) return -1;
    if (a->flat > b->flat) return 1;
    return 0;
}

/* lp: [2, T, nk] float; scores: [T, K] float; indices: [T, K] int64.  Returns 0, or -1 on bad args. */
int bf_router_topk(const float* lp, int64_t T, int nk, int K, float* scores, int64_t* indices) {
    if (!lp || T < 0 || nk <= 0 || K < 0 || (int64_t)K > (int64_t)nk * nk) return -1;
    int64_t n = (int64_t)nk * nk;
    bf_pair* all = (bf_pair*)malloc(sizeof(bf_pair) * (size_t)n);
    if (!all) return -2;
    for (int64_t t = 0; t < T; ++t) {
        const float* hx = lp + t * nk;
        const float* hy = lp + (T + t) * nk;
        for (int i = 0; i < nk; ++i)
            for (int j = 0; j < nk; ++j) {
                volatile float s = hx[i] + hy[j];   /* volatile: force a float-rounded sum */
                all[(int64_t)i * nk + j].score = s;
                all[(int64_t)i * nk + j].flat = (int64_t)i * nk + j;
            }
        qsort(all, (size_t)n, sizeof(bf_pair), bf_pair_cmp);
        for (int k = 0; k < K; ++k) {
            scores[t * K + k] = all[k].score;
            indices[t * K + k] = all[k].flat;
        }
    }
    free(all);
    return 0;
}

/*
 * x: [T, H]; wr: [2*nk, H]; logits, lp: [2, T, nk] (half-major, contiguous).
 * training != 0: batch mean / biased variance, written to mean_out/var_out (biased) when non-null.
 * training == 0: mean_in/var_in are used.
 */
int bf_prologue(const double* x, const double* wr, int64_t T, int H, int nk, int training,
                const double* mean_in, const double* var_in, double eps,
                double* mean_out, double* var_out, double* logits, double* lp) {
    double* mean = (double*)calloc((size_t)H, sizeof(double));
    double* var = (double*)calloc((size_t)H, sizeof(double));
    double* q = (double*)malloc(sizeof(double) * (size_t)H);
    if (!mean || !var || !q) return -2;
    if (training) {
        for (int64_t t = 0; t < T; ++t)
            for (int h = 0; h < H; ++h) mean[h] += x[t * H + h];
        for (int h = 0; h < H; ++h) mean[h] /= (double)T;
        for (int64_t t = 0; t < T; ++t)
            for (int h = 0; h < H; ++h) {
                double d = x[t * H + h] - mean[h];
                var[h] += d * d;
            }
        for (int h = 0; h < H; ++h) var[h] /= (double)T;
    } else {
        memcpy(mean, mean_in, sizeof(double) * (size_t)H);
        memcpy(var, var_in, sizeof(double) * (size_t)H);
    }
    if (mean_out) memcpy(mean_out, mean, sizeof(double) * (size_t)H);
    if (var_out) memcpy(var_out, var, sizeof(double) * (size_t)H);
    for (int64_t t = 0; t < T; ++t) {
        for (int h = 0; h < H; ++h) q[h] = (x[t * H + h] - mean[h]) / sqrt(var[h] + eps);
        for (int half = 0; half < 2; ++half) {
            double* lg = logits + ((int64_t)half * T + t) * nk;
            double* lq = lp + ((int64_t)half * T + t) * nk;
            double mx = -INFINITY;
            for (int n = 0; n < nk; ++n) {
                const double* wrow = wr + ((int64_t)half * nk + n) * H;
                double acc = 0.0;
                for (int h = 0; h < H; ++h) acc += q[h] * wrow[h];
                lg[n] = acc;
                if (acc > mx) mx = acc;
            }
            double z = 0.0;
            for (int n = 0; n < nk; ++n) z += exp(lg[n] - mx);
            double lz = mx + log(z);
            for (int n = 0; n < nk; ++n) lq[n] = lg[n] - lz;
        }
    }
    free(mean); free(var); free(q);
    return 0;
}

static double bf_silu(double v) { return v / (1.0 + exp(-v)); }

/* x: [T,H]; wd, wu: [E,H]; idx: [T,K]; g: [T,K]; out: [T,H] */
int bf_expert(const double* x, const double* wd, const double* wu, const int64_t* idx,
              const double* g, int64_t T, int H, int64_t E, int K, double* out) {
    for (int64_t t = 0; t < T; ++t) {
        double* o = out + t * H;
        for (int h = 0; h < H; ++h) o[h] = 0.0;
        for (int k = 0; k < K; ++k) {
            int64_t e = idx[t * K + k];
            if (e < 0 || e >= E) return -1;
            double s = 0.0;
            for (int h = 0; h < H; ++h) s += x[t * H + h] * wd[e * H + h];
            double a = bf_silu(s) * g[t * K + k];
            for (int h = 0; h < H; ++h) o[h] += a * wu[e * H + h];
        }
    }
    return 0;
}

/* x: [T,H]; wg, wu: [I,H]; wd: [H,I]; out: [T,H] */
int bf_mlp(const double* x, const double* wg, const double* wu, const double* wd,
           int64_t T, int H, int I, double* out) {
    double* hbuf = (double*)malloc(sizeof(double) * (size_t)I);
    if (!hbuf) return -2;
    for (int64_t t = 0; t < T; ++t) {
        for (int i = 0; i < I; ++i) {
            double a = 0.0, b = 0.0;
            for (int h = 0; h < H; ++h) {
                a += x[t * H + h] * wg[(int64_t)i * H + h];
                b += x[t * H + h] * wu[(int64_t)i * H + h];
            }
            hbuf[i] = bf_silu(a) * b;
        }
        for (int h = 0; h < H; ++h) {
            double acc = 0.0;
            for (int i = 0; i < I; ++i) acc += hbuf[i] * wd[(int64_t)h * I + i];
            out[t * H + h] = acc;
        }
    }
    free(hbuf);
    return 0;
}

/* Expert-centric bucketing by exhaustive scan: for every expert in turn, every pair in index order.
 * idx: [P] expert id of pair p; offsets: [E+1]; sorted_pairs: [P] (the first offsets[E] entries are written).
 * Ids outside [0,E) belong to no segment. */
int bf_bucket(const int64_t* idx, int64_t P, int64_t E, int32_t* offsets, int32_t* sorted_pairs) {
    int64_t n = 0;
    for (int64_t e = 0; e < E; ++e) {
        offsets[e] = (int32_t)n;
        for (int64_t p = 0; p < P; ++p)
            if (idx[p] == e) sorted_pairs[n++] = (int32_t)p;
    }
    offsets[E] = (int32_t)n;
    return 0;
}

/* PEER: bf_expert with the erf GELU in place of SiLU.  PKM: out[t] = sum_k w[t,k] * values[idx[t,k]]. */
int bf_peer(const double* x, const double* wd, const double* wu, const int64_t* idx,
            const double* g, int64_t T, int H, int64_t E, int K, double* out) {
    for (int64_t t = 0; t < T; ++t) {
        double* o = out + t * H;
        for (int h = 0; h < H; ++h) o[h] = 0.0;
        for (int k = 0; k < K; ++k) {
            int64_t e = idx[t * K + k];
            if (e < 0 || e >= E) return -1;
            double s = 0.0;
            for (int h = 0; h < H; ++h) s += x[t * H + h] * wd[e * H + h];
            double a = 0.5 * s * (1.0 + erf(s / sqrt(2.0))) * g[t * K + k];
            for (int h = 0; h < H; ++h) o[h] += a * wu[e * H + h];
        }
    }
    return 0;
}

int bf_pkm(const double* values, const int64_t* idx, const double* w, int64_t T, int H, int64_t E, int K, double* out) {
    for (int64_t t = 0; t < T; ++t) {
        double* o = out + t * H;
        for (int h = 0; h < H; ++h) o[h] = 0.0;
        for (int k = 0; k < K; ++k) {
            int64_t e = idx[t * K + k];
            if (e < 0 || e >= E) return -1;
            for (int h = 0; h < H; ++h) o[h] += w[t * K + k] * values[e * H + h];
        }
    }
    return 0;
}
