/*
 * C-ABI of libkge_hip.so: the MI355X (gfx950) implementation of the per-shard
 * KGE training step of graphcore/distributed-kge-poplar.
 *
 * Two groups of entry points:
 *   1. the engine: what the reference's pybind11 module binds
 *      (src/lib.cpp:46-51 -> poplar_kge::Engine, src/poplar_kge.hpp:57-75),
 *      i.e. Engine(settings, gp_folder) and Engine::run(command, data);
 *   2. the device ops: what the reference's PAG layer calls for this path
 *      (src/poplar_extensions/distance.hpp:11-36, src/pag/pag.hpp multiSlice,
 *      logSigmoid, logSoftmax, Model::getLoss, src/fructose/frnn.hpp adam),
 *      taking plain device pointers and sizes.
 *
 * Plain C types only.  All functions return a kge_status; on failure `err`
 * (if non-NULL) receives a NUL-terminated message.  The status maps back to
 * the exception type the reference throws at the same place:
 *   KGE_INVALID_ARGUMENT  std::invalid_argument  (src/poplar_kge.cpp:39-106, 130-134, ...)
 *   KGE_RUNTIME_ERROR     std::runtime_error     (device attach, HIP failures)
 *   KGE_LOGIC_ERROR       std::logic_error
 */
#ifndef KGE_HIP_H
#define KGE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct kge_engine kge_engine;

typedef enum {
    KGE_OK = 0,
    KGE_INVALID_ARGUMENT = 1,
    KGE_RUNTIME_ERROR = 2,
    KGE_LOGIC_ERROR = 3
} kge_status;

/* One entry of the reference's `Batch` map (src/poplar_kge.hpp:38-50):
 * string | ArrayView<float> | ArrayView<uint32_t> | ArrayView<float16> |
 * bool | float | unsigned | map<string,float>.  Arrays are HOST pointers to
 * C-contiguous data that the caller keeps alive for the call; outputs are
 * written in place (src/poplar_kge.hpp:17-31). */
typedef enum {
    KGE_STR = 0,
    KGE_F32 = 1,
    KGE_U32 = 2,
    KGE_F16 = 3,
    KGE_BOOL = 4,
    KGE_FLOAT = 5,
    KGE_UINT = 6,
    KGE_MAP = 7
} kge_kind;

typedef struct kge_item {
    const char* key;
    int kind;                     /* kge_kind */
    void* data;                   /* KGE_F32 / KGE_U32 / KGE_F16 */
    const size_t* shape;
    size_t rank;
    double num;                   /* KGE_BOOL / KGE_FLOAT / KGE_UINT */
    const char* str;              /* KGE_STR */
    const char* const* map_keys;  /* KGE_MAP */
    const float* map_vals;
    size_t map_len;
} kge_item;

/* Replaces poplar_kge::Engine::Engine(const Batch& settings, const std::string&
 * gpFolder) (src/poplar_kge.cpp:1001-1002 -> EngineImpl::create :919-948).
 * `settings` holds the flattened dotted keys read at src/poplar_kge.cpp:198-236.
 * `gp_folder` is accepted for signature compatibility and ignored (there are no
 * codelet files to load). */
int kge_engine_create(const kge_item* settings, size_t n_settings, const char* gp_folder,
                      kge_engine** out, char* err, size_t err_len);

/* Replaces poplar_kge::Engine::run(const std::string& command, Batch& data)
 * (src/poplar_kge.cpp:950-965, 1004-1006).  Commands, with the reference's item
 * names, dtypes and shapes (every array has the leading n_shard axis S):
 *   "train_step_loop"  learning_rate f32[S], loss f32[S] (out), remote
 *                      u32[S, n_step, B + S*A], a2a u32[S, n_step, S, A], head /
 *                      relation / tail u32[S, n_step, B]      (:713-720, 740)
 *   "predict"          predict_head, predict_relation u32[S, Hb],
 *                      predict_entity_count u32[S]; out predict_scores f32 and
 *                      predict_indices u32 [S, S, Hb, n_best]  (:812-855)
 *   "read_entity"      read_indices u32[S, rw], read_data [S, rw, 3D+F] (out)
 *   "write_entity"     write_indices u32[S, rw], write_features [S, rw, F]
 *   "read" / "write"   name (string), value (the variable's shape)  (:977-991)
 *   "variables"        served by the two functions below, because its result is
 *                      a list and not an array                      (:993-998)
 * Additive commands, not in the reference: "write_entity_raw" (full rows from
 * the host), "stage_batch" + "train_step_loop" with {"staged": true} (keeps the
 * index arrays resident in HBM), "gather_benchmark", "timing", "plan_dump" (the
 * distinct rows, segments and sorted items the device derived for one step). */
int kge_engine_run(kge_engine* engine, const char* command, kge_item* items, size_t n_items,
                   char* err, size_t err_len);

/* Replaces EngineImpl::runVariables (src/poplar_kge.cpp:993-998): the list of
 * (name, shape) with the leading dimension multiplied by n_shard
 * (src/poplar_kge.cpp:306-318). */
size_t kge_engine_variable_count(const kge_engine* engine);
int kge_engine_variable_info(const kge_engine* engine, size_t index, const char** name,
                             const size_t** shape, size_t* rank);

void kge_engine_destroy(kge_engine* engine);

/* ---- device ops ---------------------------------------------------------
 * All pointers are DEVICE pointers, row-major float32 unless noted; `stream`
 * is a hipStream_t (NULL = the default stream).  The calls are asynchronous. */

/* poplar_extensions::l1distance / l2distance (distance.hpp:11-15, 24-28):
 * out[m,n] = sum_k |a[m,k]-b[n,k]|  /  sqrt(sum_k (a[m,k]-b[n,k])^2).
 * kge_dot_score: pag::ops::matMul(a, b^T) (src/pag/pag.cpp:673-683). */
int kge_l1_distance(const float* a, const float* b, float* out, int M, int N, int D, void* stream);
int kge_l2_distance(const float* a, const float* b, float* out, int M, int N, int D, void* stream);
int kge_dot_score(const float* a, const float* b, float* out, int M, int N, int D, void* stream);

/* poplar_extensions::l1distancegrad / l2distancegrad (distance.hpp:17-22,
 * 30-36): gradient of the FIRST operand,
 *   grad[m,k] = sum_n g[m,n] * signum(a[m,k]-b[n,k])              (L1)
 *   grad[m,k] = sum_n g[m,n] * (a[m,k]-b[n,k]) / dist[m,n], 0 at dist==0 (L2)
 * g and dist are [M,N].  The second operand's gradient is the same call with
 * the operands swapped and g, dist transposed (src/pag/pag.cpp:787-801,
 * 821-831). */
int kge_l1_distance_grad(const float* a, const float* b, const float* g, float* grad, int M, int N,
                         int D, void* stream);
int kge_l2_distance_grad(const float* a, const float* b, const float* dist, const float* g,
                         float* grad, int M, int N, int D, void* stream);

/* fr::Buffer::read / write (src/fructose/fructose.cpp:790-806): indexed row
 * copies out[i,:] = buf[idx[i],:] and buf[idx[i],:] = data[i,:];
 * row_bytes must be a multiple of 4. */
int kge_buffer_read(const void* buf, const uint32_t* idx, void* out, int64_t n, int64_t row_bytes,
                    void* stream);
int kge_buffer_write(void* buf, const uint32_t* idx, const void* data, int64_t n,
                     int64_t row_bytes, void* stream);

/* pag::ops::multiSlice backward = popops::multiUpdateAdd into a zeroed table
 * (src/pag/pag.cpp:721-743): grad_t[r,:] = sum over i with idx[i] == r of
 * grad_out[i,:] -- every row of grad_t is overwritten (rows nobody indexes
 * become zero, as the reference's zeroed table leaves them), duplicates are
 * summed deterministically (sort by index + segmented reduce).  `workspace`
 * must hold kge_scatter_add_workspace_bytes(n, rows, cols) bytes (16-byte aligned).
 * Indices are expected in [0, rows); an index outside that range adds nothing (its
 * gradient row is dropped, no row of grad_t is touched by it) where the reference
 * would address memory outside the table.  n + rows must be below 2^31. */
size_t kge_scatter_add_workspace_bytes(int64_t n, int64_t rows, int64_t cols);
int kge_scatter_add(float* grad_t, int64_t rows, int64_t cols, const uint32_t* idx, int64_t n,
                    const float* grad_out, void* workspace, void* stream);

/* kge_scatter_add for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same arguments and results as kge_scatter_add,
 * without the workspace: it lives in a fixed array of
 * kge_scatter_add_static_max_bytes() bytes (16 MiB) that every GPU the library
 * runs on holds until the process ends.  Sizes whose workspace
 * (kge_scatter_add_workspace_bytes) exceeds that are rejected with
 * KGE_INVALID_ARGUMENT and a message in `err`.  The call allocates and frees
 * nothing (the runtime itself sets a stream's queue up, scratch for the kernels'
 * private segments included, when kernels first run on that stream: issue one
 * call on the stream beforehand where even that matters).  All calls on one GPU
 * share that GPU's array: calls that overlap in
 * time on one GPU (different streams, or host threads) race; issue them in
 * order on one stream. */
size_t kge_scatter_add_static_max_bytes(void);
int kge_scatter_add_static(float* grad_t, int64_t rows, int64_t cols, const uint32_t* idx, int64_t n,
                           const float* grad_out, void* stream, char* err, size_t err_len);

/* fr::nn::adam (src/fructose/frnn.cpp:61-90), fused, in place.  With
 * v_is_sqrt != 0 the third array holds sqrt(v) as the entity rows do
 * (src/poplar_kge.cpp:695-703). */
int kge_adam(float* p, float* m, float* v, const float* g, int64_t n, float alpha, float beta_m,
             float beta_v, float epsilon, float weight_decay, int v_is_sqrt, void* stream);

/* pag::ops::logSigmoid forward and backward (src/pag/pag.cpp:888-910, with its
 * clamps at -11 / +11): y[i] = logsigmoid(x[i]), dx[i] = dy[i] * d logsigmoid /
 * dx (dy NULL: 1; y or dx NULL: not stored).  form 0 evaluates the two
 * functions as the row-wise loss kernel does, form 1 as the scoring kernels'
 * fused epilogue does (one hardware exponential for both). */
int kge_log_sigmoid(const float* x, const float* dy, float* y, float* dx, int64_t n, int form,
                    void* stream);

/* pag::ops::logSoftmax over the last axis (src/pag/pag.cpp:841-852) and its
 * backward dx = dy - exp(y) * sum(dy) (:853-859); [rows, cols] row-major. */
int kge_log_softmax(const float* x, float* y, int64_t rows, int64_t cols, void* stream);
int kge_log_softmax_grad(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols,
                         void* stream);

/* Model::getLoss (src/poplar_kge.cpp:615-660) on the score matrices of S shards,
 * by the kernel the training step runs for the softmax and the adversarial
 * loss: score f32[S, B, T] (T = S * a2a_size), label u32[S, B] (position of the
 * true tail in the row).  loss_fn 0 logsigmoid (weights :617-622, self-
 * adversarial weighting :623-633 when negative_adversarial_scale > 0), 1 softmax
 * (softmax_correction = correction_weight * (log(n_entity*S - 1) - log(T - 1)),
 * :640-650).  Outputs: loss f32[S] per shard, row_loss f32[S, B] its per-positive
 * terms, dscore f32[S, B, T] = loss_scale * d loss / d score (dscore may alias
 * score). */
int kge_loss(int loss_fn, const float* score, const uint32_t* label, int S, int B, int T,
             float softmax_correction, float negative_adversarial_scale, float loss_scale,
             float* loss, float* row_loss, float* dscore, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KGE_HIP_H */
