/*
 * CPU oracle for the per-shard KGE training step.  TEST INFRASTRUCTURE ONLY:
 * nothing on the product path may link, load or call this file; it exists so
 * that tests, the smoke check and the bench's cpu_baseline leg have an
 * independent restatement of the reference arithmetic to compare against.
 *
 * Every function restates one piece of graphcore/distributed-kge-poplar and
 * cites the file:line it follows (paths relative to the reference checkout).
 * The arithmetic type is the macro REAL: the build makes two libraries from
 * this one source, REAL=double ("truth", summation order irrelevant) and
 * REAL=float (sequential fp32 sums, the same order the reference's non-IPU
 * codelets use; also the timed CPU baseline).  Storage (tables, variables,
 * inputs, outputs) is always float32 exactly as the reference streams it.
 *
 * Parity pinning (see tests/test_oracle_kat.py): every op below is checked
 * against the reference's own inline known-answer vectors
 * (tests/pag/testPag.cpp, tests/fructose/testFructose.cpp,
 * tests/testPoplarKge.cpp), against torch autograd / closed forms, and the
 * whole step against an independent torch-autograd restatement (every score
 * function incl. ComplEx, whose restatement there is torch.complex arithmetic,
 * plus a closed-form Re<h r, conj t> check in numpy).  The one option that is
 * not the reference's, cfg.scoring_bf16 (operands of the scoring and projection
 * products rounded to bfloat16, float32 accumulation), is pinned the same way
 * with a straight-through rounding in the autograd restatement.
 * "parity unpinned": RotatE's float16 sine and cosine only.  The reference takes them with
 * the IPU's float16 instructions, whose last-bit rounding no fixture here records; this
 * file (and the torch restatement, with torch's float16 kernels) round the correctly
 * rounded float result to float16.  Everything around them -- the float16 cast of the
 * phases, the rotation, the float16 gradient arithmetic -- is pinned against autograd.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REAL
#define REAL double
#endif

#define API __attribute__((visibility("default")))

enum { SCORE_TRANSE = 0, SCORE_DISTMULT = 1, SCORE_COMPLEX = 2, SCORE_ROTATE = 3, SCORE_TRANSH = 4 };
enum { DIST_L1 = 0, DIST_L2 = 1, DIST_DOT = 2 };
enum { LOSS_LOGSIGMOID = 0, LOSS_SOFTMAX = 1 };
enum { STORE_F32 = 0, STORE_F16 = 1, STORE_BF16_EMB = 2 };

typedef struct {
    int32_t n_shard;        /* S: replicas (virtual shards / blocks)            */
    int32_t n_entity;       /* rows per shard table, row 0 = padding            */
    int32_t n_relation;     /* nRel (whole table, all shards)                   */
    int32_t dim;            /* D                                                */
    int32_t feature;        /* F                                                */
    int32_t batch;          /* B positives per shard                            */
    int32_t a2a;            /* A tails sent to each shard; T = S*A              */
    int32_t score_fn;       /* SCORE_*                                          */
    int32_t distance_fn;    /* DIST_* (ignored for DistMult, which is a dot)    */
                            /* ComplEx: dim even; score = distance_fn's value   */
    int32_t loss_fn;        /* LOSS_*                                           */
    int32_t shared_table;   /* 1: every shard addresses the same n_entity rows  */
    int32_t storage;        /* STORE_*: rounding applied on row write-back      */
    int32_t mlp_size;       /* M > 0: feature MLP (poplar_kge.cpp:453-458), the feature part of
                             * hidden is relu([embedding | feature . W] . Up) . Down with
                             * Up [2D, M], Down [M, D]; `proj` and its moments then hold
                             * W, Up and Down back to back                               */
    int32_t scoring_bf16;   /* 1: predicted tails and tails rounded to bfloat16
                             * before the dot product, features and projection
                             * before theirs (products exact, sums in REAL);
                             * gradients pass straight through the rounding      */
    float gamma;
    float beta_m, beta_v, epsilon, weight_decay;
    float loss_scale;
    float softmax_correction_weight;
    float negative_adversarial_scale;
    float lr_mod_entity, lr_mod_relation, lr_mod_projection;
    /* norm regularisers (poplar_kge.cpp:430-437, 463-465): weight * sum over the gathered
     * rows of (sum_k |x_k^power|)^(1/power), of the embedding, of feature . W and of
     * their sum; weight 0 = off                                                          */
    float reg_emb_power, reg_emb_weight, reg_feat_power, reg_feat_weight, reg_hid_power, reg_hid_weight;
    /* feature dropout (poplar_kge.cpp:459-461; pag.cpp:596-617): the feature part of hidden times
     * a keep mask / (1 - p), drawn separately for the rows' use as heads and as tails.  The
     * reference's device random stream cannot be matched; the mask here is kge_dropout_keep, a
     * hash of (seed, step, role, table row, column) that the HIP kernels evaluate identically. */
    float dropout;
    uint32_t dropout_seed;
    /* 1: separate feature networks for a row's use as a head and as a tail
     * (share_feature_networks = false, poplar_kge.cpp:268-273): `proj` and its moments hold the
     * head network's parameters, then the tail network's                                      */
    int32_t separate_networks;
} kge_oracle_cfg;

/* keep (1) or drop (0) element k of table row `key` in `role` (0 head, 1 tail) at optimiser step
 * `step`: a 32-bit integer hash compared with p * 2^32 */
API int kge_dropout_keep(uint32_t seed, uint32_t step, uint32_t role, uint32_t key, uint32_t k, float p) {
    uint32_t x = key * 0x9E3779B1u + k * 0x85EBCA77u + role * 0xC2B2AE3Du + step * 0x27D4EB2Fu + seed * 0x165667B1u;
    x ^= x >> 16; x *= 0x7FEB352Du; x ^= x >> 15; x *= 0x846CA68Bu; x ^= x >> 16;
    return x >= (uint32_t)((double)p * 4294967296.0);
}

/* ------------------------------------------------------------------------ */
/* lpnorm (poplar_kge.cpp:389-391): pow(sum(abs(pow(a, p))), 1/p) of one row, and its
 * gradient through the reference's pow / abs backward ops (pag.cpp:483-503, 440-459):
 *   d pow(x, e) = g * e * pow(x, e) / (x + (x == 0))     (0 at x = 0)
 *   d abs(x)    = g * signum(x)
 * which multiply out to  g * (n / s) * |a_k^p| / a_k  (0 where a_k = 0 or s = 0).
 * Adds g * that to grad[0..D) (grad may be NULL) and returns n.                      */
static REAL lpnorm_row(const REAL* a, int64_t D, float power, REAL g, REAL* grad) {
    REAL s = 0;
    for (int64_t k = 0; k < D; ++k) s += (REAL)fabs(pow((double)a[k], (double)power));
    const REAL n = (REAL)pow((double)s, 1.0 / (double)power);
    if (grad && s != 0)
        for (int64_t k = 0; k < D; ++k)
            if (a[k] != 0) grad[k] += g * (n / s) * (REAL)fabs(pow((double)a[k], (double)power)) / a[k];
    return n;
}

/* ------------------------------------------------------------------------ */
/* storage rounding helpers (write-back cast, poplar_kge.cpp:412-417)        */

static float round_bf16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return x; /* NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    memcpy(&x, &u, 4);
    return x;
}

static float round_f16(float x) {
    /* float32 -> IEEE binary16 -> float32, round-to-nearest-even, by bit
     * manipulation (gcc 11 has no _Float16 on x86-64). */
    uint32_t u;
    memcpy(&u, &x, 4);
    const uint32_t sign = u & 0x80000000u;
    uint32_t mag = u & 0x7fffffffu;
    if (mag >= 0x7f800000u) return x;                    /* inf / NaN */
    if (mag >= 0x477ff000u) {                            /* >= 65520 rounds to inf */
        u = sign | 0x7f800000u;
        memcpy(&x, &u, 4);
        return x;
    }
    if (mag < 0x38800000u) {                             /* below 2^-14: half subnormal grid 2^-24 */
        const float q = 16777216.0f;                     /* 2^24 */
        float a = fabsf(x) * q;
        a = nearbyintf(a);                               /* RNE in the default rounding mode */
        a /= q;
        return sign ? -a : a;
    }
    mag += 0xfffu + ((mag >> 13) & 1u);                  /* RNE at 13 dropped mantissa bits */
    mag &= 0xffffe000u;
    u = sign | mag;
    memcpy(&x, &u, 4);
    return x;
}

API float kge_oracle_round(float x, int storage_kind) {
    if (storage_kind == STORE_F16) return round_f16(x);
    if (storage_kind == STORE_BF16_EMB) return round_bf16(x);
    return x;
}

/* ------------------------------------------------------------------------ */
/* Row gather / write-back: fr::Buffer::read / write
 * (src/fructose/fructose.cpp:790-806): out[i,:] = buf[idx[i],:] and
 * buf[idx[i],:] = data[i,:] (later duplicates overwrite earlier ones).     */

API void kge_oracle_buffer_read(const float* buf, int64_t row, const uint32_t* idx, int64_t n,
                                float* out) {
    for (int64_t i = 0; i < n; ++i) memcpy(out + i * row, buf + (int64_t)idx[i] * row, row * 4);
}

API void kge_oracle_buffer_write(float* buf, int64_t row, const uint32_t* idx, int64_t n,
                                 const float* data) {
    for (int64_t i = 0; i < n; ++i) memcpy(buf + (int64_t)idx[i] * row, data + i * row, row * 4);
}

/* Slot gather and its backward, pag::ops::multiSlice
 * (src/pag/pag.cpp:706-746): fwd out[i] = t[idx[i]]; bwd zero then
 * grad_t[idx[i]] += grad_out[i] with duplicates summed (multiUpdateAdd,
 * scale 1.0).                                                              */

API void kge_oracle_multi_slice(const float* t, int64_t cols, const uint32_t* idx, int64_t n,
                                float* out) {
    for (int64_t i = 0; i < n; ++i) memcpy(out + i * cols, t + (int64_t)idx[i] * cols, cols * 4);
}

API void kge_oracle_multi_update_add(float* grad_t, int64_t rows, int64_t cols, const uint32_t* idx,
                                     int64_t n, const float* grad_out) {
    REAL* acc = (REAL*)calloc((size_t)(rows * cols), sizeof(REAL));
    for (int64_t i = 0; i < n; ++i)
        for (int64_t k = 0; k < cols; ++k) acc[(int64_t)idx[i] * cols + k] += grad_out[i * cols + k];
    for (int64_t i = 0; i < rows * cols; ++i) grad_t[i] = (float)acc[i];
    free(acc);
}

/* ------------------------------------------------------------------------ */
/* L1 distance: src/poplar_extensions/l1distance.codelet.cpp:47-56 (fwd),
 * :76-79 signum with signum(0)=0, :136-145 (grad of the first operand:
 * grad[m,k] = sum_n g[m,n] * signum(a[m,k]-b[n,k])).  The second operand's
 * gradient is the same routine with operands swapped and g transposed
 * (src/pag/pag.cpp:787-801).                                               */

static REAL signum(REAL x) { return (REAL)((0 < x) - (x < 0)); }

API void kge_oracle_l1_distance(const float* a, const float* b, int64_t M, int64_t N, int64_t D,
                                float* out) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            REAL s = 0;
            for (int64_t k = 0; k < D; ++k) s += (REAL)fabs((REAL)a[m * D + k] - (REAL)b[n * D + k]);
            out[m * N + n] = (float)s;
        }
}

API void kge_oracle_l1_distance_grad(const float* a, const float* b, const float* g, int64_t M,
                                     int64_t N, int64_t D, float* grad_a) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < D; ++k) {
            REAL s = 0;
            for (int64_t n = 0; n < N; ++n)
                s += (REAL)g[m * N + n] * signum((REAL)a[m * D + k] - (REAL)b[n * D + k]);
            grad_a[m * D + k] = (float)s;
        }
}

/* L2 distance: src/poplar_extensions/l2distance.codelet.cpp:52-62 (fwd
 * sqrt(sum (a-b)^2)), :147-158 (grad[m,k] = sum_n g[m,n]*(a[m,k]-b[n,k])/
 * dist[m,n], the term being 0 where dist==0; uses the SAVED forward dist,
 * src/pag/pag.cpp:821-831).                                                */

API void kge_oracle_l2_distance(const float* a, const float* b, int64_t M, int64_t N, int64_t D,
                                float* out) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            REAL s = 0;
            for (int64_t k = 0; k < D; ++k) {
                REAL d = (REAL)a[m * D + k] - (REAL)b[n * D + k];
                s += d * d;
            }
            out[m * N + n] = (float)sqrt((double)s);
        }
}

API void kge_oracle_l2_distance_grad(const float* a, const float* b, const float* dist,
                                     const float* g, int64_t M, int64_t N, int64_t D,
                                     float* grad_a) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < D; ++k) {
            REAL s = 0;
            for (int64_t n = 0; n < N; ++n) {
                REAL dn = dist[m * N + n];
                if (dn != 0) s += (REAL)g[m * N + n] * ((REAL)a[m * D + k] - (REAL)b[n * D + k]) / dn;
            }
            grad_a[m * D + k] = (float)s;
        }
}

/* Dot-product score and its two gradients, pag::ops::matMul
 * (src/pag/pag.cpp:673-704): S = A * B^T; dA = G * B; dB = G^T * A.         */

API void kge_oracle_dot_score(const float* a, const float* b, int64_t M, int64_t N, int64_t D,
                              float* out) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            REAL s = 0;
            for (int64_t k = 0; k < D; ++k) s += (REAL)a[m * D + k] * (REAL)b[n * D + k];
            out[m * N + n] = (float)s;
        }
}

/* ------------------------------------------------------------------------ */
/* logSigmoid, src/pag/pag.cpp:888-910:
 *   y  = x > -11 ? -log1p(exp(-max(x,-11))) : x
 *   dx = dy / (1 + exp(min(x, 11)))                                         */

static REAL log_sigmoid(REAL x) { return x > -11 ? -(REAL)log1p(exp(-(double)(x > -11 ? x : -11))) : x; }
static REAL log_sigmoid_grad(REAL x) { return 1 / (1 + (REAL)exp((double)(x < 11 ? x : 11))); }

API void kge_oracle_log_sigmoid(const float* x, int64_t n, float* y) {
    for (int64_t i = 0; i < n; ++i) y[i] = (float)log_sigmoid(x[i]);
}
API void kge_oracle_log_sigmoid_grad(const float* x, const float* dy, int64_t n, float* dx) {
    for (int64_t i = 0; i < n; ++i) dx[i] = (float)((REAL)dy[i] * log_sigmoid_grad(x[i]));
}

/* logSoftmax over the last axis, src/pag/pag.cpp:841-864:
 *   y = x - logsumexp(x);  dx = dy - sum(dy) * exp(y)                       */

API void kge_oracle_log_softmax(const float* x, int64_t rows, int64_t cols, float* y) {
    for (int64_t r = 0; r < rows; ++r) {
        REAL mx = x[r * cols];
        for (int64_t c = 1; c < cols; ++c) mx = x[r * cols + c] > mx ? x[r * cols + c] : mx;
        REAL s = 0;
        for (int64_t c = 0; c < cols; ++c) s += (REAL)exp((double)((REAL)x[r * cols + c] - mx));
        REAL lse = mx + (REAL)log((double)s);
        for (int64_t c = 0; c < cols; ++c) y[r * cols + c] = (float)((REAL)x[r * cols + c] - lse);
    }
}
API void kge_oracle_log_softmax_grad(const float* y, const float* dy, int64_t rows, int64_t cols,
                                     float* dx) {
    for (int64_t r = 0; r < rows; ++r) {
        REAL s = 0;
        for (int64_t c = 0; c < cols; ++c) s += dy[r * cols + c];
        for (int64_t c = 0; c < cols; ++c)
            dx[r * cols + c] = (float)((REAL)dy[r * cols + c] - s * (REAL)exp((double)y[r * cols + c]));
    }
}

/* fr::nn::softmaxCrossEntropy, src/fructose/frnn.cpp:18-23:
 *   xent[r] = -logsoftmax(logits)[r, label[r]]                              */
API void kge_oracle_softmax_cross_entropy(const float* logits, const uint32_t* labels, int64_t rows,
                                          int64_t cols, float* xent) {
    float* y = (float*)malloc((size_t)(rows * cols) * 4);
    kge_oracle_log_softmax(logits, rows, cols, y);
    for (int64_t r = 0; r < rows; ++r) xent[r] = -y[r * cols + labels[r]];
    free(y);
}

/* detachedSoftmax = popnn SOFTMAX_STABLE over the last axis,
 * src/poplar_kge.cpp:905-912.                                               */
API void kge_oracle_softmax(const float* x, int64_t rows, int64_t cols, float* y) {
    for (int64_t r = 0; r < rows; ++r) {
        REAL mx = x[r * cols];
        for (int64_t c = 1; c < cols; ++c) mx = x[r * cols + c] > mx ? x[r * cols + c] : mx;
        REAL s = 0;
        for (int64_t c = 0; c < cols; ++c) s += (REAL)exp((double)((REAL)x[r * cols + c] - mx));
        for (int64_t c = 0; c < cols; ++c)
            y[r * cols + c] = (float)((REAL)exp((double)((REAL)x[r * cols + c] - mx)) / s);
    }
}

/* ------------------------------------------------------------------------ */
/* Adam: fr::nn::adamStepSizeAutoIncrement (src/fructose/frnn.cpp:42-59):
 *   step += 1; alpha = lr * sqrt(1 - beta_v^step) / (1 - beta_m^step)
 * fr::nn::adam (src/fructose/frnn.cpp:61-90):
 *   m = beta_m m + (1-beta_m) g;  v = beta_v v + (1-beta_v) g g
 *   p = p - alpha (m / (sqrt(v) + eps) + wd p)
 * Entity rows hold sqrt(v): v is squared before and square-rooted after
 * (src/poplar_kge.cpp:695-703).                                            */

API float kge_oracle_adam_step_size(uint32_t* step, float lr, float beta_m, float beta_v) {
    *step += 1;
    double num = sqrt(1.0 - pow((double)beta_v, (double)*step));
    double den = 1.0 - pow((double)beta_m, (double)*step);
    return (float)((REAL)(num / den) * (REAL)lr);
}

API void kge_oracle_adam(float* p, float* m, float* v, const float* g, int64_t n, float alpha,
                         float beta_m, float beta_v, float eps, float wd, int v_is_sqrt) {
    for (int64_t i = 0; i < n; ++i) {
        REAL vi = v[i];
        if (v_is_sqrt) vi = vi * vi;
        REAL gi = g[i];
        REAL mi = (REAL)beta_m * (REAL)m[i] + (REAL)(1 - beta_m) * gi;
        vi = (REAL)beta_v * vi + (REAL)(1 - beta_v) * gi * gi;
        REAL pi = p[i];
        pi = pi - (REAL)alpha * (mi / ((REAL)sqrt((double)vi) + (REAL)eps) + (REAL)wd * pi);
        p[i] = (float)pi;
        m[i] = (float)mi;
        v[i] = v_is_sqrt ? (float)sqrt((double)vi) : (float)vi;
    }
}

/* ------------------------------------------------------------------------ */
/* Loss forward + d(loss)/d(score), Model::getLoss (src/poplar_kge.cpp:615-660).
 * score[B,T], label[B] in [0,T).  Returns the shard loss; writes
 * dscore = d(loss)/d(score) (NOT yet multiplied by the loss scale).         */

static REAL shard_loss(const kge_oracle_cfg* c, const REAL* score, const uint32_t* label,
                       REAL* dscore) {
    const int64_t S = c->n_shard, B = c->batch, A = c->a2a, T = S * A;
    REAL loss = 0;
    if (c->loss_fn == LOSS_LOGSIGMOID) {
        /* :617-636 */
        const REAL w_neg = ((REAL)0.5 * T) / (T - 1), w_pos = (REAL)0.5 * T;
        const REAL norm = (REAL)(S * B * A * S);
        REAL* adv = NULL;
        if (c->negative_adversarial_scale > 0) adv = (REAL*)malloc(sizeof(REAL) * (size_t)T);
        for (int64_t b = 0; b < B; ++b) {
            if (adv) { /* :623-633, detached stable softmax of alpha*s - 1e4*onehot */
                REAL mx = -INFINITY, sum = 0;
                for (int64_t t = 0; t < T; ++t) {
                    adv[t] = (REAL)c->negative_adversarial_scale * score[b * T + t] +
                             (t == label[b] ? (REAL)-10000 : 0);
                    mx = adv[t] > mx ? adv[t] : mx;
                }
                for (int64_t t = 0; t < T; ++t) sum += (REAL)exp((double)(adv[t] - mx));
                for (int64_t t = 0; t < T; ++t) adv[t] = (REAL)exp((double)(adv[t] - mx)) / sum;
            }
            for (int64_t t = 0; t < T; ++t) {
                const int pos = (t == label[b]);
                REAL w = pos ? w_pos : w_neg; /* (w_pos-w_neg)*onehot + w_neg */
                if (adv) w *= (pos ? 1 : 0) + (REAL)(T - 1) * adv[t];
                const REAL sign = pos ? 1 : -1;
                const REAL z = sign * score[b * T + t];
                loss += -w * log_sigmoid(z) / norm;
                dscore[b * T + t] = -w * sign * log_sigmoid_grad(z) / norm;
            }
        }
        free(adv);
    } else {
        /* :638-652, softmax cross entropy with the flat-sampling correction */
        REAL corr = 0;
        if (c->softmax_correction_weight != 0)
            corr = (REAL)(c->softmax_correction_weight *
                          (float)(log((double)((int64_t)c->n_entity * S - 1)) -
                                  log((double)(S * A - 1))));
        const REAL norm = (REAL)(S * B);
        for (int64_t b = 0; b < B; ++b) {
            REAL mx = -INFINITY, sum = 0;
            for (int64_t t = 0; t < T; ++t) {
                REAL z = score[b * T + t] + (t == label[b] ? 0 : corr);
                mx = z > mx ? z : mx;
            }
            for (int64_t t = 0; t < T; ++t) {
                REAL z = score[b * T + t] + (t == label[b] ? 0 : corr);
                sum += (REAL)exp((double)(z - mx));
            }
            const REAL lse = mx + (REAL)log((double)sum);
            for (int64_t t = 0; t < T; ++t) {
                REAL z = score[b * T + t] + (t == label[b] ? 0 : corr);
                REAL p = (REAL)exp((double)(z - lse));
                if (t == label[b]) loss += -(z - lse) / norm;
                dscore[b * T + t] = (p - (t == label[b] ? 1 : 0)) / norm;
            }
        }
    }
    return loss;
}

/* Standalone entry so tests can pin the loss against an independent
 * restatement (tests/python/reference_model.py:126-152).                    */
API float kge_oracle_loss(const kge_oracle_cfg* c, const float* score, const uint32_t* label,
                          float* dscore) {
    const int64_t n = (int64_t)c->batch * c->n_shard * c->a2a;
    REAL* s = (REAL*)malloc(sizeof(REAL) * (size_t)n);
    REAL* d = (REAL*)malloc(sizeof(REAL) * (size_t)n);
    for (int64_t i = 0; i < n; ++i) s[i] = score[i];
    REAL loss = shard_loss(c, s, label, d);
    for (int64_t i = 0; i < n; ++i) dscore[i] = (float)d[i];
    free(s);
    free(d);
    return (float)loss;
}

/* ------------------------------------------------------------------------ */
/* One training step, Model::trainStep (src/poplar_kge.cpp:664-707).
 *
 * table      f32[n_tables * n_entity, 3D+F]   stacked rows [emb|m|sqrt v|feat]
 *            (n_tables = 1 if shared_table else S), :274-275
 * rel,*_m,*_v f32[nRel, D]   relation_embedding and its Adam moments (true v)
 * proj,*_m,*_v f32[F, D]     feature_projection likewise (ignored if F == 0)
 * step       u32, incremented (one counter; every shard's copy is equal)
 * lr         f32[S]          per-shard learning rate; shard s's rows and
 *                            shard s's slice of each dense parameter use lr[s]
 * remote u32[S, B+T], a2a u32[S,S,A], head/relation/tail u32[S,B], :713-720
 * loss_out   f32[S]          per-shard loss of this step
 *
 * Duplicate rows (the same table row in several shards' `remote` when the
 * table is shared, or repeated padding zeros) get ONE Adam update with the
 * sum of all their slots' gradients; with unique `remote` per shard and
 * private tables this is exactly the reference.                            */

/* Test hook: when set, every training step also stores the gradients its updates are made from
 * (after the scatter-add over duplicate slots, times the loss scale; later steps overwrite):
 * ent[key * D + k] for every gathered table row, rel[r * RD + k] for every relation row.     */
static double* g_tap_ent = NULL;
static double* g_tap_rel = NULL;
API void kge_oracle_gradient_tap(double* ent, double* rel) { g_tap_ent = ent; g_tap_rel = rel; }

static int cmp_u64(const void* a, const void* b) {
    uint64_t x = *(const uint64_t*)a, y = *(const uint64_t*)b;
    return (x > y) - (x < y);
}

API int kge_oracle_train_step(const kge_oracle_cfg* c, float* table, float* rel, float* rel_m,
                              float* rel_v, float* proj, float* proj_m, float* proj_v,
                              uint32_t* step, const float* lr, const uint32_t* remote,
                              const uint32_t* a2a, const uint32_t* head, const uint32_t* relation,
                              const uint32_t* tail, float* loss_out) {
    const int64_t S = c->n_shard, B = c->batch, A = c->a2a, T = S * A, NR = B + T;
    const int64_t D = c->dim, F = c->feature, ROW = 3 * D + F, NREL = c->n_relation;
    /* RotatE's relation rows are D / 2 phases (poplar_kge.cpp:248-249) */
    const int64_t RD = c->score_fn == SCORE_ROTATE ? D / 2 : D;
    const int64_t NE = c->n_entity;
    /* TransH (poplar_kge.cpp:252-255): `rel` and its moments hold 2 * NREL rows, the
     * relation embeddings followed by the hyperplane normals (relation_normal)       */
    const int transh = c->score_fn == SCORE_TRANSH;
    const int64_t M = F > 0 ? c->mlp_size : 0;
    /* one feature network = W [F, D], Up [2D, M], Down [M, D] back to back */
    const int64_t NETSIZE = F * D + 3 * D * M;
    const int nets = (F > 0 && c->separate_networks) ? 2 : 1;
    const int64_t NRELT = transh ? 2 * NREL : NREL;
#define KEY(s, slot) ((c->shared_table ? 0 : (int64_t)(s) * NE) + (int64_t)remote[(s) * NR + (slot)])

    /* 1. gather + hidden = emb + feature part (:405-410, :439-467).  entityHidden runs once for
     * the rows' use as heads and once for their use as tails (:676-678).  The two differ when
     * the feature networks are separate or with dropout (masks drawn per call): then a slot has
     * two hidden rows (`hidden`, `hidden_t`) and two gradients (`ghid`, `ghid_t`); otherwise
     * these are the same arrays.                                                              */
    const int drop = F > 0 && c->dropout > 0;
    const int n_role = (drop || nets == 2) ? 2 : 1;
    const REAL keep_scale = drop ? 1 / (1 - (REAL)c->dropout) : 1;
    REAL* hidden = (REAL*)malloc(sizeof(REAL) * (size_t)(S * NR * D));
    REAL* ghid = (REAL*)calloc((size_t)(S * NR * D), sizeof(REAL));
    REAL* hidden_t = n_role == 2 ? (REAL*)malloc(sizeof(REAL) * (size_t)(S * NR * D)) : hidden;
    REAL* ghid_t = n_role == 2 ? (REAL*)calloc((size_t)(S * NR * D), sizeof(REAL)) : ghid;
    /* per role: the projected features (second half of the MLP's input) and the MLP's
     * pre-activations, kept for the backward pass; whether the dropout's output is non-zero
     * (what its backward tests)                                                               */
    REAL *fproj_r[2] = {NULL, NULL}, *pre_r[2] = {NULL, NULL};
    uint8_t* live_r[2] = {NULL, NULL};
    REAL* fhv = (REAL*)malloc(sizeof(REAL) * (size_t)D); /* one slot's feature part of hidden */
    for (int role = 0; role < n_role; ++role) {
        const float* W = proj + (nets == 2 ? role : 0) * NETSIZE;
        const float* up = W + F * D;          /* [2D, M] */
        const float* down = up + 2 * D * M;   /* [M, D]  */
        REAL* hid = role ? hidden_t : hidden;
        if (M) {
            fproj_r[role] = (REAL*)calloc((size_t)(S * NR * D), sizeof(REAL));
            pre_r[role] = (REAL*)calloc((size_t)(S * NR * M), sizeof(REAL));
        }
        if (drop) live_r[role] = (uint8_t*)malloc((size_t)(S * NR * D));
        for (int64_t s = 0; s < S; ++s)
            for (int64_t j = 0; j < NR; ++j) {
                const float* row = table + KEY(s, j) * ROW;
                REAL* h = hid + (s * NR + j) * D;
                REAL* fh = M ? fproj_r[role] + (s * NR + j) * D : fhv; /* feature . W */
                for (int64_t k = 0; k < D; ++k) fhv[k] = 0;
                for (int64_t f = 0; f < F; ++f) {
                    /* bfloat16 scoring also takes the projection's operands in bfloat16 */
                    const REAL x = c->scoring_bf16 ? round_bf16(row[3 * D + f]) : row[3 * D + f];
                    if (x != 0)
                        for (int64_t k = 0; k < D; ++k)
                            fh[k] += x * (REAL)(c->scoring_bf16 ? round_bf16(W[f * D + k]) : W[f * D + k]);
                }
                if (M) { /* :453-458: boom = relu(concat(value, featureHidden) . Up); featureHidden = boom . Down */
                    REAL* a = pre_r[role] + (s * NR + j) * M;
                    for (int64_t i = 0; i < 2 * D; ++i) {
                        const REAL x = i < D ? (REAL)row[i] : fh[i - D];
                        for (int64_t m = 0; m < M; ++m) a[m] += x * (REAL)up[i * M + m];
                    }
                    for (int64_t m = 0; m < M; ++m)
                        if (a[m] > 0)
                            for (int64_t k = 0; k < D; ++k) fhv[k] += a[m] * (REAL)down[m * D + k];
                }
                if (drop) { /* :459-461: keep mask / (1 - p), a draw of its own for every call */
                    const uint32_t key = (uint32_t)KEY(s, j);
                    for (int64_t k = 0; k < D; ++k) {
                        const int keep = kge_dropout_keep(c->dropout_seed, *step, (uint32_t)role, key, (uint32_t)k,
                                                          c->dropout);
                        const REAL o = keep ? fhv[k] * keep_scale : 0;
                        h[k] = (REAL)row[k] + o;
                        live_r[role][(s * NR + j) * D + k] = o != 0;
                    }
                } else {
                    for (int64_t k = 0; k < D; ++k) h[k] = (REAL)row[k] + fhv[k]; /* :462 */
                }
            }
    }
    free(fhv);

    /* 1b. norm regularisers over every gathered slot (:463-465).  entityHidden runs once for
     * the heads and once for the tails on the same gathered rows (:676-678), so every term
     * counts twice; when the two runs differ (separate networks, dropout) each run's feature
     * part and hidden row are regularised once.  The embedding's gradient (greg_val) and the
     * feature part's gradient per run (greg_fh_r) differ from here on.                        */
    const int reg_on = c->reg_emb_weight > 0 || c->reg_feat_weight > 0 || c->reg_hid_weight > 0;
    REAL* greg_val = reg_on ? (REAL*)calloc((size_t)(S * NR * D), sizeof(REAL)) : NULL;
    REAL* greg_fh_r[2] = {NULL, NULL};
    REAL* reg_loss = (REAL*)calloc((size_t)S, sizeof(REAL));
    if (reg_on) {
        REAL* fh = (REAL*)malloc(sizeof(REAL) * (size_t)D);
        REAL* val = (REAL*)malloc(sizeof(REAL) * (size_t)D);
        REAL* tmp = (REAL*)malloc(sizeof(REAL) * (size_t)D);
        const REAL uses = n_role == 2 ? 1 : 2; /* runs of entityHidden one pass of this loop stands for */
        for (int role = 0; role < n_role; ++role) {
            greg_fh_r[role] = (REAL*)calloc((size_t)(S * NR * D), sizeof(REAL));
            for (int64_t s = 0; s < S; ++s)
                for (int64_t j = 0; j < NR; ++j) {
                    const float* row = table + KEY(s, j) * ROW;
                    const REAL* h = (role ? hidden_t : hidden) + (s * NR + j) * D;
                    REAL* gv = greg_val + (s * NR + j) * D;
                    REAL* gf = greg_fh_r[role] + (s * NR + j) * D;
                    for (int64_t k = 0; k < D; ++k) { val[k] = row[k]; fh[k] = h[k] - val[k]; }
                    const REAL seed = uses * (REAL)c->loss_scale;
                    if (c->reg_emb_weight > 0) {
                        for (int64_t k = 0; k < D; ++k) tmp[k] = 0;
                        reg_loss[s] += uses * c->reg_emb_weight *
                                       lpnorm_row(val, D, c->reg_emb_power, seed * c->reg_emb_weight, tmp);
                        for (int64_t k = 0; k < D; ++k) gv[k] += tmp[k];
                    }
                    if (c->reg_feat_weight > 0) {
                        for (int64_t k = 0; k < D; ++k) tmp[k] = 0;
                        reg_loss[s] += uses * c->reg_feat_weight *
                                       lpnorm_row(fh, D, c->reg_feat_power, seed * c->reg_feat_weight, tmp);
                        for (int64_t k = 0; k < D; ++k) gf[k] += tmp[k];
                    }
                    if (c->reg_hid_weight > 0) {
                        for (int64_t k = 0; k < D; ++k) tmp[k] = 0;
                        reg_loss[s] += uses * c->reg_hid_weight *
                                       lpnorm_row(h, D, c->reg_hid_power, seed * c->reg_hid_weight, tmp);
                        for (int64_t k = 0; k < D; ++k) { gv[k] += tmp[k]; gf[k] += tmp[k]; }
                    }
                }
        }
        free(fh); free(val); free(tmp);
    }

    REAL* grel = (REAL*)calloc((size_t)(NRELT * RD), sizeof(REAL));
    /* TransH: unit normals of the positives, their gradient, norms of the raw normals */
    REAL* nv = transh ? (REAL*)malloc(sizeof(REAL) * (size_t)(B * D)) : NULL;
    REAL* dnv = transh ? (REAL*)malloc(sizeof(REAL) * (size_t)(B * D)) : NULL;
    REAL* nrm = transh ? (REAL*)malloc(sizeof(REAL) * (size_t)B) : NULL;
    REAL* p = (REAL*)malloc(sizeof(REAL) * (size_t)(B * D));
    REAL* tl = (REAL*)malloc(sizeof(REAL) * (size_t)(T * D));
    REAL* score = (REAL*)malloc(sizeof(REAL) * (size_t)(B * T));
    REAL* dist = (REAL*)malloc(sizeof(REAL) * (size_t)(B * T));
    REAL* dscore = (REAL*)malloc(sizeof(REAL) * (size_t)(B * T));
    REAL* dp = (REAL*)malloc(sizeof(REAL) * (size_t)(B * D));
    REAL* dtl = (REAL*)malloc(sizeof(REAL) * (size_t)(T * D));

    for (int64_t d = 0; d < S; ++d) {
        /* 2. heads / predicted tails (:676-677, :488-490, :567-569) */
        for (int64_t b = 0; b < B; ++b) {
            const REAL* h = hidden + (d * NR + head[d * B + b]) * D;
            const float* r = rel + (int64_t)relation[d * B + b] * RD;
            if (c->score_fn == SCORE_ROTATE) {
                /* rotatEPredict (:516-530): the phases pass through float16, as do their sine
                 * and cosine, which then rotate (h_re, h_im) in float32 */
                const int64_t H = D / 2;
                for (int64_t k = 0; k < H; ++k) {
                    const float th = round_f16(r[k]);
                    const REAL sn = round_f16((float)sin((double)th)), cs = round_f16((float)cos((double)th));
                    p[b * D + k] = h[k] * cs - h[k + H] * sn;
                    p[b * D + k + H] = h[k + H] * cs + h[k] * sn;
                }
                continue;
            }
            if (transh) {
                /* transHPredict (:539-549): unit normal, head projected onto the hyperplane,
                 * plus the relation embedding; the normal travels on to the score */
                const float* w = rel + (NREL + (int64_t)relation[d * B + b]) * D;
                REAL ss = 0, a = 0;
                for (int64_t k = 0; k < D; ++k) ss += (REAL)w[k] * (REAL)w[k];
                nrm[b] = (REAL)sqrt((double)ss);
                for (int64_t k = 0; k < D; ++k) nv[b * D + k] = (REAL)w[k] / nrm[b];
                for (int64_t k = 0; k < D; ++k) a += nv[b * D + k] * h[k];
                for (int64_t k = 0; k < D; ++k) p[b * D + k] = (h[k] - nv[b * D + k] * a) + (REAL)r[k];
                continue;
            }
            if (c->score_fn == SCORE_COMPLEX) {
                /* complExPredict (:501-510): halves are real | imaginary parts, (h_re + i h_im)(r_re + i r_im) */
                const int64_t H = D / 2;
                for (int64_t k = 0; k < H; ++k) {
                    p[b * D + k] = h[k] * (REAL)r[k] - h[k + H] * (REAL)r[k + H];
                    p[b * D + k + H] = h[k] * (REAL)r[k + H] + h[k + H] * (REAL)r[k];
                }
                continue;
            }
            for (int64_t k = 0; k < D; ++k)
                p[b * D + k] = c->score_fn == SCORE_TRANSE ? h[k] + (REAL)r[k] : h[k] * (REAL)r[k];
        }
        /* tails after the all-to-all (:678-681): block j of shard d's tails
         * is what shard j gathered with a2a[j][d][:]                        */
        for (int64_t j = 0; j < S; ++j)
            for (int64_t i = 0; i < A; ++i)
                memcpy(tl + (j * A + i) * D, hidden_t + (j * NR + a2a[(j * S + d) * A + i]) * D,
                       sizeof(REAL) * (size_t)D);

        if (c->scoring_bf16) {
            for (int64_t x = 0; x < B * D; ++x) p[x] = (REAL)round_bf16((float)p[x]);
            for (int64_t x = 0; x < T * D; ++x) tl[x] = (REAL)round_bf16((float)tl[x]);
        }

        /* 3. scores (:492-499, :571-573, :469-486) */
        const int dot = (c->score_fn == SCORE_DISTMULT) || c->distance_fn == DIST_DOT;
        for (int64_t b = 0; b < B; ++b)
            for (int64_t t = 0; t < T; ++t) {
                REAL acc = 0;
                const REAL *x = p + b * D, *y = tl + t * D;
                if (transh) {
                    /* transHScore (:551-565): tails projected onto the positive's hyperplane,
                     * L1 distance whatever distance_fn says */
                    const REAL* n = nv + b * D;
                    REAL cn = 0;
                    for (int64_t k = 0; k < D; ++k) cn += n[k] * y[k];
                    for (int64_t k = 0; k < D; ++k) acc += (REAL)fabs((double)(x[k] - (y[k] - n[k] * cn)));
                } else if (dot)
                    for (int64_t k = 0; k < D; ++k) acc += x[k] * y[k];
                else if (c->distance_fn == DIST_L1)
                    for (int64_t k = 0; k < D; ++k) acc += (REAL)fabs((double)(x[k] - y[k]));
                else {
                    for (int64_t k = 0; k < D; ++k) acc += (x[k] - y[k]) * (x[k] - y[k]);
                    acc = (REAL)sqrt((double)acc);
                }
                dist[b * T + t] = acc;
                /* distMultScore / complExScore return the distance function's value itself
                 * (:512-514, :571-573); TransE gamma minus it (:492-499) */
                if (c->score_fn == SCORE_DISTMULT || c->score_fn == SCORE_COMPLEX)
                    score[b * T + t] = acc;
                else
                    score[b * T + t] = (REAL)c->gamma - acc;
            }

        /* 4. loss + backward seed = loss_scale (:688-691) */
        loss_out[d] = (float)(shard_loss(c, score, tail + d * B, dscore) + reg_loss[d]);  /* :688 */
        for (int64_t i = 0; i < B * T; ++i) dscore[i] *= (REAL)c->loss_scale;

        /* 5. backward through the score into p and tails */
        memset(dp, 0, sizeof(REAL) * (size_t)(B * D));
        memset(dtl, 0, sizeof(REAL) * (size_t)(T * D));
        if (transh) memset(dnv, 0, sizeof(REAL) * (size_t)(B * D));
        for (int64_t b = 0; b < B; ++b)
            for (int64_t t = 0; t < T; ++t) {
                const REAL *x = p + b * D, *y = tl + t * D;
                REAL* gx = dp + b * D;
                REAL* gy = dtl + t * D;
                REAL g = dscore[b * T + t];
                if (transh) {
                    /* e = p - (tail - n c), c = n . tail: abs, sub, mul, matMul backward in turn */
                    const REAL* n = nv + b * D;
                    REAL* gn = dnv + b * D;
                    REAL cn = 0, gc = 0;
                    g = -g;
                    for (int64_t k = 0; k < D; ++k) cn += n[k] * y[k];
                    for (int64_t k = 0; k < D; ++k) {
                        const REAL u = g * signum(x[k] - (y[k] - n[k] * cn));
                        gx[k] += u;         /* predicted tail */
                        gy[k] -= u;         /* projected tail -> tail */
                        gn[k] += u * cn;    /* projected tail -> normal * c */
                        gc += u * n[k];     /* ... -> c */
                    }
                    for (int64_t k = 0; k < D; ++k) {
                        gn[k] += gc * y[k];
                        gy[k] += gc * n[k];
                    }
                    continue;
                }
                if (c->score_fn == SCORE_DISTMULT) { /* pag.cpp:685-700 */
                    for (int64_t k = 0; k < D; ++k) {
                        gx[k] += g * y[k];
                        gy[k] += g * x[k];
                    }
                    continue;
                }
                if (c->score_fn == SCORE_TRANSE || c->score_fn == SCORE_ROTATE)
                    g = -g; /* score = gamma - distance (pag.cpp sub: :323-345) */
                if (dot) {
                    for (int64_t k = 0; k < D; ++k) {
                        gx[k] += g * y[k];
                        gy[k] += g * x[k];
                    }
                } else if (c->distance_fn == DIST_L1) {
                    for (int64_t k = 0; k < D; ++k) {
                        const REAL sg = signum(x[k] - y[k]);
                        gx[k] += g * sg;
                        gy[k] -= g * sg;
                    }
                } else {
                    const REAL dn = dist[b * T + t];
                    if (dn != 0)
                        for (int64_t k = 0; k < D; ++k) {
                            const REAL u = g * (x[k] - y[k]) / dn;
                            gx[k] += u;
                            gy[k] -= u;
                        }
                }
            }

        /* backward through predictTail and the slot gathers (multiUpdateAdd) */
        for (int64_t b = 0; b < B; ++b) {
            REAL* gh = ghid + (d * NR + head[d * B + b]) * D;
            const REAL* h = hidden + (d * NR + head[d * B + b]) * D;
            const int64_t r = relation[d * B + b];
            if (transh) {
                /* p = h - n (n . h) + rel;  n = w / |w| */
                const REAL *n = nv + b * D, *gp = dp + b * D;
                REAL* gn = dnv + b * D;
                REAL a = 0, sgn = 0, ngn = 0;
                for (int64_t k = 0; k < D; ++k) { a += n[k] * h[k]; sgn += gp[k] * n[k]; }
                for (int64_t k = 0; k < D; ++k) {
                    gh[k] += gp[k] - n[k] * sgn;
                    grel[r * D + k] += gp[k];
                    gn[k] += -a * gp[k] - h[k] * sgn;
                }
                for (int64_t k = 0; k < D; ++k) ngn += n[k] * gn[k];
                for (int64_t k = 0; k < D; ++k) grel[(NREL + r) * D + k] += (gn[k] - n[k] * ngn) / nrm[b];
                continue;
            }
            if (c->score_fn == SCORE_ROTATE) {
                /* p_re = h_re cos - h_im sin, p_im = h_im cos + h_re sin.  The gradient of the
                 * phase runs in float16 as the forward does (cast's backward casts the gradient,
                 * pag.cpp:619-637; sin' = g cos, cos' = -g sin, :552-594), then back to float32 */
                const int64_t H = D / 2;
                for (int64_t k = 0; k < H; ++k) {
                    const REAL gre = dp[b * D + k], gim = dp[b * D + k + H];
                    const float th = round_f16(rel[r * RD + k]);
                    const float sn = round_f16((float)sin((double)th)), cs = round_f16((float)cos((double)th));
                    gh[k] += gre * cs + gim * sn;
                    gh[k + H] += gim * cs - gre * sn;
                    const float g_sin = round_f16((float)(-gre * h[k + H] + gim * h[k]));
                    const float g_cos = round_f16((float)(gre * h[k] + gim * h[k + H]));
                    /* backward ops run in reverse: cos's first, then sin's is added to it */
                    const float from_cos = round_f16((float)(-(double)g_cos * (double)sn));
                    const float from_sin = round_f16((float)((double)g_sin * (double)cs));
                    grel[r * RD + k] += (REAL)round_f16((float)((double)from_cos + (double)from_sin));
                }
                continue;
            }
            if (c->score_fn == SCORE_COMPLEX) {
                /* p_re = h_re r_re - h_im r_im, p_im = h_re r_im + h_im r_re */
                const int64_t H = D / 2;
                for (int64_t k = 0; k < H; ++k) {
                    const REAL gre = dp[b * D + k], gim = dp[b * D + k + H];
                    const REAL rre = rel[r * D + k], rim = rel[r * D + k + H];
                    gh[k] += gre * rre + gim * rim;
                    gh[k + H] += gim * rre - gre * rim;
                    grel[r * D + k] += gre * h[k] + gim * h[k + H];
                    grel[r * D + k + H] += gim * h[k] - gre * h[k + H];
                }
                continue;
            }
            for (int64_t k = 0; k < D; ++k) {
                if (c->score_fn == SCORE_TRANSE) {
                    gh[k] += dp[b * D + k];
                    grel[r * D + k] += dp[b * D + k];
                } else {
                    gh[k] += dp[b * D + k] * (REAL)rel[r * D + k];
                    grel[r * D + k] += dp[b * D + k] * h[k];
                }
            }
        }
        for (int64_t j = 0; j < S; ++j)
            for (int64_t i = 0; i < A; ++i) {
                REAL* gh = ghid_t + (j * NR + a2a[(j * S + d) * A + i]) * D;
                for (int64_t k = 0; k < D; ++k) gh[k] += dtl[(j * A + i) * D + k];
            }
    }

    /* 6. step size (:692-693); one alpha per shard because lr is per shard */
    float* alpha = (float*)malloc(sizeof(float) * (size_t)S);
    {
        uint32_t st = *step;
        for (int64_t s = 0; s < S; ++s) {
            st = *step;
            alpha[s] = kge_oracle_adam_step_size(&st, lr[s], c->beta_m, c->beta_v);
        }
        *step = st;
    }

    /* feature-projection gradient: dW = sum_slots feature^T ghid (matMul bwd,
     * pag.cpp:694-700; hidden is built for head and tail from the same W
     * when the networks are shared, so the two uses' gradients add up to
     * the per-slot ghid already accumulated above)                          */
    REAL* gproj = NULL;
    REAL* gmlp_val = NULL; /* feature MLP: what reaches the embedding through the MLP's input */
    if (F > 0) {
        gproj = (REAL*)calloc((size_t)(nets * NETSIZE), sizeof(REAL));
        REAL* gfh = (REAL*)malloc(sizeof(REAL) * (size_t)D);
        REAL* gpre = M ? (REAL*)malloc(sizeof(REAL) * (size_t)M) : NULL;
        if (M) gmlp_val = (REAL*)calloc((size_t)(S * NR * D), sizeof(REAL));
        for (int role = 0; role < n_role; ++role) {
            const int net = nets == 2 ? role : 0;
            const float* W = proj + net * NETSIZE;
            const float* up = W + F * D;
            const float* down = up + 2 * D * M;
            REAL* gW = gproj + net * NETSIZE;
            REAL* gup = gW + F * D;
            REAL* gdown = gup + 2 * D * M;
            const REAL* gsrc = role ? ghid_t : ghid;
            for (int64_t s = 0; s < S; ++s)
                for (int64_t j = 0; j < NR; ++j) {
                    const float* row = table + KEY(s, j) * ROW;
                    const REAL* gh = gsrc + (s * NR + j) * D;
                    const REAL* gr = greg_fh_r[role] ? greg_fh_r[role] + (s * NR + j) * D : NULL;
                    for (int64_t k = 0; k < D; ++k) gfh[k] = gh[k] + (gr ? gr[k] : 0);
                    if (drop) { /* grad * (output != 0) / (1 - p) (pag.cpp:606-614) */
                        const uint8_t* lv = live_r[role] + (s * NR + j) * D;
                        for (int64_t k = 0; k < D; ++k) gfh[k] = lv[k] ? keep_scale * gfh[k] : 0;
                    }
                    if (M) {
                        /* matMul, max(., 0) (its gradient passes where input == output, i.e. also at
                         * exactly 0: pag.cpp:650-658), matMul, concat backward in turn */
                        const REAL* a = pre_r[role] + (s * NR + j) * M;
                        const REAL* fh = fproj_r[role] + (s * NR + j) * D;
                        REAL* gv = gmlp_val + (s * NR + j) * D;
                        for (int64_t m = 0; m < M; ++m) {
                            const REAL boom = a[m] > 0 ? a[m] : 0;
                            REAL acc = 0;
                            for (int64_t k = 0; k < D; ++k) {
                                gdown[m * D + k] += boom * gfh[k];
                                acc += gfh[k] * (REAL)down[m * D + k];
                            }
                            gpre[m] = a[m] >= 0 ? acc : 0;
                        }
                        for (int64_t i = 0; i < 2 * D; ++i) {
                            const REAL x = i < D ? (REAL)row[i] : fh[i - D];
                            REAL acc = 0;
                            for (int64_t m = 0; m < M; ++m) {
                                gup[i * M + m] += x * gpre[m];
                                acc += gpre[m] * (REAL)up[i * M + m];
                            }
                            if (i < D) gv[i] += acc; else gfh[i - D] = acc;
                        }
                    }
                    for (int64_t f = 0; f < F; ++f) {
                        const REAL x = c->scoring_bf16 ? round_bf16(row[3 * D + f]) : row[3 * D + f];
                        if (x != 0)
                            for (int64_t k = 0; k < D; ++k) gW[f * D + k] += x * gfh[k];
                    }
                }
        }
        free(gfh); free(gpre);
    }

    /* 7. entity Adam on every gathered row, one update per distinct row
     * (:695-704).  Sort (key, slot) so duplicates are adjacent.             */
    {
        const int64_t n = S * NR;
        uint64_t* ks = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)n);
        for (int64_t s = 0; s < S; ++s)
            for (int64_t j = 0; j < NR; ++j)
                ks[s * NR + j] = ((uint64_t)KEY(s, j) << 24) | (uint64_t)(s * NR + j);
        qsort(ks, (size_t)n, sizeof(uint64_t), cmp_u64);
        REAL* g = (REAL*)malloc(sizeof(REAL) * (size_t)D);
        float* gf = (float*)malloc(sizeof(float) * (size_t)D);
        for (int64_t i = 0; i < n;) {
            const int64_t key = (int64_t)(ks[i] >> 24);
            memset(g, 0, sizeof(REAL) * (size_t)D);
            int64_t j = i;
            for (; j < n && (int64_t)(ks[j] >> 24) == key; ++j) {
                const REAL* gh = ghid + (int64_t)(ks[j] & 0xffffff) * D;
                const REAL* gr = greg_val ? greg_val + (int64_t)(ks[j] & 0xffffff) * D : NULL;
                const REAL* gm = gmlp_val ? gmlp_val + (int64_t)(ks[j] & 0xffffff) * D : NULL;
                const REAL* gt = n_role == 2 ? ghid_t + (int64_t)(ks[j] & 0xffffff) * D : NULL;
                for (int64_t k = 0; k < D; ++k)
                    g[k] += gh[k] + (gt ? gt[k] : 0) + (gr ? gr[k] : 0) + (gm ? gm[k] : 0);
            }
            for (int64_t k = 0; k < D; ++k) gf[k] = (float)g[k];
            if (g_tap_ent) for (int64_t k = 0; k < D; ++k) g_tap_ent[key * D + k] = (double)g[k];
            float* row = table + key * ROW;
            const int64_t shard = c->shared_table ? 0 : key / NE;
            kge_oracle_adam(row, row + D, row + 2 * D, gf, D, alpha[shard] * c->lr_mod_entity,
                            c->beta_m, c->beta_v, c->epsilon, c->weight_decay, /*v_is_sqrt*/ 1);
            if (c->storage == STORE_BF16_EMB)
                for (int64_t k = 0; k < D; ++k) row[k] = round_bf16(row[k]);
            if (c->storage == STORE_F16)
                for (int64_t k = 0; k < 3 * D; ++k) row[k] = round_f16(row[k]);
            i = j;
        }
        free(ks);
        free(g);
        free(gf);
    }

    /* 8. dense Adam on the SRAM parameters (:329-339): every row, every step;
     * shard s owns rows [s*n/S, (s+1)*n/S) of each parameter (:290-304)     */
    {
        float* gf = (float*)malloc(sizeof(float) * (size_t)D);
        for (int64_t r = 0; r < NRELT; ++r) {
            for (int64_t k = 0; k < RD; ++k) gf[k] = (float)grel[r * RD + k];
            if (g_tap_rel) for (int64_t k = 0; k < RD; ++k) g_tap_rel[r * RD + k] = (double)grel[r * RD + k];
            const int64_t shard = c->shared_table ? 0 : (r % NREL) / (NREL / S);
            kge_oracle_adam(rel + r * RD, rel_m + r * RD, rel_v + r * RD, gf, RD,
                            alpha[shard] * c->lr_mod_relation, c->beta_m, c->beta_v, c->epsilon,
                            c->weight_decay, 0);
        }
        free(gf);
        /* the feature networks' matrices, rows split over the shards like every parameter; the
         * MLP's have no step-size modifier of their own here */
        for (int net = 0; net < nets && F > 0; ++net) {
            const int64_t base = net * NETSIZE;
            const int64_t off[3] = {base, base + F * D, base + F * D + 2 * D * M};
            const int64_t rows[3] = {F, M ? 2 * D : 0, M}, width[3] = {D, M, D};
            for (int q = 0; q < 3; ++q) {
                if (rows[q] == 0) continue;
                float* gw = (float*)malloc(sizeof(float) * (size_t)width[q]);
                for (int64_t r = 0; r < rows[q]; ++r) {
                    const int64_t o = off[q] + r * width[q];
                    for (int64_t k = 0; k < width[q]; ++k) gw[k] = (float)gproj[o + k];
                    const int64_t shard = c->shared_table ? 0 : r / (rows[q] / S);
                    kge_oracle_adam(proj + o, proj_m + o, proj_v + o, gw, width[q],
                                    alpha[shard] * (q == 0 ? c->lr_mod_projection : 1.0f), c->beta_m, c->beta_v,
                                    c->epsilon, c->weight_decay, 0);
                }
                free(gw);
            }
        }
    }
#undef KEY
    free(greg_val); free(greg_fh_r[0]); free(greg_fh_r[1]); free(reg_loss);
    free(hidden); free(ghid); free(grel); free(p); free(tl); free(score); free(dist);
    free(dscore); free(dp); free(dtl); free(alpha); free(gproj);
    free(nv); free(dnv); free(nrm); free(gmlp_val);
    for (int role = 0; role < 2; ++role) { free(fproj_r[role]); free(pre_r[role]); free(live_r[role]); }
    if (n_role == 2) { free(hidden_t); free(ghid_t); }
    return 0;
}

/* Model::trainStepLoop (src/poplar_kge.cpp:709-741): n_step steps over
 * inputs with a leading [S, n_step] layout as the host passes them
 * (remote u32[S,n_step,B+T], a2a u32[S,n_step,S,A], head/relation/tail
 * u32[S,n_step,B]); loss_out[s] = mean over steps of shard s's loss.        */
API int kge_oracle_train_step_loop(const kge_oracle_cfg* c, int32_t n_step, float* table, float* rel,
                                   float* rel_m, float* rel_v, float* proj, float* proj_m,
                                   float* proj_v, uint32_t* step, const float* lr,
                                   const uint32_t* remote, const uint32_t* a2a, const uint32_t* head,
                                   const uint32_t* relation, const uint32_t* tail, float* loss_out) {
    const int64_t S = c->n_shard, B = c->batch, A = c->a2a, T = S * A, NR = B + T;
    uint32_t* r1 = (uint32_t*)malloc(4 * (size_t)(S * NR));
    uint32_t* a1 = (uint32_t*)malloc(4 * (size_t)(S * S * A));
    uint32_t* h1 = (uint32_t*)malloc(4 * (size_t)(S * B));
    uint32_t* q1 = (uint32_t*)malloc(4 * (size_t)(S * B));
    uint32_t* t1 = (uint32_t*)malloc(4 * (size_t)(S * B));
    float* l1 = (float*)malloc(4 * (size_t)S);
    double* tot = (double*)calloc((size_t)S, sizeof(double));
    for (int32_t i = 0; i < n_step; ++i) {
        for (int64_t s = 0; s < S; ++s) {
            memcpy(r1 + s * NR, remote + (s * n_step + i) * NR, 4 * (size_t)NR);
            memcpy(a1 + s * S * A, a2a + (s * n_step + i) * S * A, 4 * (size_t)(S * A));
            memcpy(h1 + s * B, head + (s * n_step + i) * B, 4 * (size_t)B);
            memcpy(q1 + s * B, relation + (s * n_step + i) * B, 4 * (size_t)B);
            memcpy(t1 + s * B, tail + (s * n_step + i) * B, 4 * (size_t)B);
        }
        kge_oracle_train_step(c, table, rel, rel_m, rel_v, proj, proj_m, proj_v, step, lr, r1, a1,
                              h1, q1, t1, l1);
        for (int64_t s = 0; s < S; ++s) tot[s] += l1[s];
    }
    for (int64_t s = 0; s < S; ++s) loss_out[s] = (float)(tot[s] / n_step);
    free(r1); free(a1); free(h1); free(q1); free(t1); free(l1); free(tot);
    return 0;
}
