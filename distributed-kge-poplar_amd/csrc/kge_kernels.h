// Internal launcher interface between the engine (host logic) and the gfx950
// kernels.  Everything here takes device pointers; nothing allocates.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace kge {

// TransE: score = gamma - distance(h + r, t).  DistMult: score = (h * r) . t.  ComplEx: the
// complex product of h and r on the (real | imaginary) halves of the row, scored by the
// distance function's value itself (src/poplar_kge.cpp:501-514).
// RotatE: (h_re, h_im) rotated by the relation's D/2 phases, whose sine and cosine pass
// through float16 as in the reference (src/poplar_kge.cpp:516-537); score = gamma - distance.
enum { SCORE_TRANSE = 0, SCORE_DISTMULT = 1, SCORE_COMPLEX = 2, SCORE_ROTATE = 3, SCORE_TRANSH = 4 };
// whether the score is the distance function's value itself (else gamma minus it)
__host__ __device__ inline bool score_is_distance_value(int score_fn) { return score_fn == SCORE_DISTMULT || score_fn == SCORE_COMPLEX; }
enum { DIST_L1 = 0, DIST_L2 = 1, DIST_DOT = 2 };
enum { LOSS_LOGSIGMOID = 0, LOSS_SOFTMAX = 1 };
enum { ET_F32 = 0, ET_BF16 = 1, ET_F16 = 2 };

constexpr int kSortTile = 4096;  // items per workgroup in one radix pass
constexpr int kScoreTile = 64;   // score tile edge (rows of either operand)

// Indexed rows: logical row r is `count` elements of type `etype` starting at
// base + index[r] * pitch (bytes).
struct RowSource {
    const char* base;
    int64_t pitch;
    int etype;
    const uint32_t* index;  // null: identity
    int count;              // elements per row
    int vec;                // rows 16-byte aligned and count % 4 == 0: float4 access allowed
};

// ---- plan phase (index-only work, batched over the steps of one call) ----

struct PlanShape {
    int n_step, S, B, A, NR;  // NR = B + S*A slots per shard
    int n_entity;             // rows per shard table
    int shared_table;
    int n_relation;
    int rel_copies;           // 1; 2 for TransH, whose relation table holds a second row (the
                              // hyperplane normal, row n_relation + r) per relation
    int step0, step_count;    // the steps of the resident batch to plan
    // the index arrays lie step by step: step i's remote [S, NR], a2a [S, S, A], head, relation and
    // tail [S, B] start idx_step_stride words behind step i - 1's (the pointers handed to the
    // launchers are step 0's)
    int64_t idx_step_stride;
    int merge_tails;          // the blocks' tail lists have been merged (launch_merge_tails)
};

// Sort keys carry one flag bit under the row number: key = row << 1 | (0: the item is a
// gradient contribution, 1: a zero-gradient member of the update set).  Within a row the
// contributions therefore sort in front, whatever their item numbers.
constexpr int kKeyFlagBits = 1;

// A block's T shared tails repeat rows under power-law sampling (a third of them on the
// benchmark workloads), and equal rows give equal score columns.  One workgroup per (step,
// block) sorts the block's tail rows and keeps one column per distinct row:
//   tkey   [n_step, S*T]  sort key of tail column j of block d (row << 1; columns from the
//                         block's distinct count on repeat column 0's row with the flag bit set:
//                         they are scored in whole tiles but carry no gradient)
//   tmult  [n_step, S*T]  how many of the block's tail positions hold column j's row (0 from the
//                         distinct count on)
//   tcol   [n_step, S*T]  the column of every original tail position (labels are positions)
//   tcount [n_step, S]    distinct rows per block
// T <= kMergeMaxT.  Integer work: exact, independent of scheduling.
constexpr int kMergeMaxT = 4096;
void launch_merge_tails(const PlanShape& ps, const uint32_t* remote, const uint32_t* a2a, uint32_t* tkey,
                        float* tmult, uint32_t* tcol, uint32_t* tcount, hipStream_t stream);

// Compact per-step arrays + the items to sort for the entity plan and the
// relation plan.  Item layout, entity plan (2R items, R = S*NR):
//   [0, S*B)          head contributions  c = d*B + b
//   [S*B, R)          tail contributions  c = S*B + d*T + (j*A + i)
//   [R, 2R)           every remote slot, as a zero-gradient member of the update set
// relation plan (S*B + n_relation items): head contributions, then every relation id; with
// rel_copies = 2 both parts twice, the second copies keyed n_relation + r (item S*B + c is the
// normal row's contribution of positive c).
// `digit_bits`: the width of the first radix pass (sort_passes of the wider of the two key
// widths); ent_hist / rel_hist receive every tile's digit histogram for that pass.
// With ps.merge_tails the tail items take their keys from `tkey` and the labels go through `tcol`.
void launch_build_items(const PlanShape& ps, const uint32_t* remote, const uint32_t* a2a,
                        const uint32_t* head, const uint32_t* relation, const uint32_t* tail,
                        const uint32_t* tkey, const uint32_t* tcol,
                        uint32_t* ckey, uint32_t* crel, uint32_t* clabel, uint32_t* ent_keys,
                        uint32_t* ent_vals, uint32_t* rel_keys, uint32_t* rel_vals, int digit_bits,
                        uint32_t* ent_hist, uint32_t* rel_hist, hipStream_t stream);

// Stable LSD radix sort of n_seg independent arrays of N (key, value) pairs on
// the low `key_bits` bits, in sort_passes(key_bits).n passes of at most kSortMaxBits bits.
// Result is in keys_a/vals_a if the return value is 0, in keys_b/vals_b if it is 1.
// hist must hold radix_sort_hist_words(N, n_seg, key_bits) words.
constexpr int kSortMaxBits = 11;
struct SortPasses { int n; int bits[4]; int shift[4]; };
SortPasses sort_passes(int key_bits);
size_t radix_sort_hist_words(int N, int n_seg, int key_bits);
int launch_radix_sort(uint32_t* keys_a, uint32_t* vals_a, uint32_t* keys_b, uint32_t* vals_b,
                      uint32_t* hist, int N, int n_seg, int key_bits, hipStream_t stream);

// Two such sorts in shared launches (the wider key's pass schedule; `schedule_bits` in the
// histogram size: radix_sort_hist_words(N, n_seg, max of the two key widths) words per job).
struct SortBuffers {
    uint32_t *keys_a, *vals_a, *keys_b, *vals_b, *hist;
    int N, key_bits;
    int result_in_b;   // out: 1 if the sorted pairs are in keys_b / vals_b
};
struct SortJob {       // one job of one pass, as the kernels see it
    uint32_t *keys_in, *vals_in, *keys_out, *vals_out, *hist;
    int N, n_tiles;
};
void launch_radix_sort2(SortBuffers* j0, SortBuffers* j1, int n_seg, bool first_hist_done, hipStream_t stream);

// Per-segment outputs of the segment finder, all with a per-step stride.
struct SegPlan {
    uint32_t* uniq_key;   // [n_seg, u_stride]      key of each distinct row, ascending
    uint32_t* seg_start;  // [n_seg, u_stride + 1]  first sorted position of each row
    uint32_t* chunk_off;  // [n_seg, u_stride + 1]  first chunk of each row
    uint32_t* chunk_pos;  // [n_seg, c_stride]      first sorted position of each chunk
    uint32_t* chunk_len;  // [n_seg, c_stride]      real items in the chunk (<= chunk size)
    uint32_t* counts;     // [n_seg, 2]             {distinct rows, chunks}
    uint32_t* item_row;   // [n_seg, n_real] or null: distinct-row index of each real item
    uint32_t* seg_real;   // [n_seg, u_stride]      real items of each row
    // or null: the rows that get chunks (more than direct_max real items), as distinct-row
    // indices in ascending order [n_seg, c_stride], and [n_seg, 2] {how many, real items of the
    // row with the most}
    uint32_t* hot_rows;
    uint32_t* hot_count;
    uint32_t* chunk_row = nullptr;  // or null: [n_seg, c_stride] distinct-row index of each chunk
    // or null: [n_seg, 4] {distinct rows, chunks, rows with chunks, real items of the biggest row}
    // once more, in device-visible host memory (the host sizes its launches from them)
    uint32_t* host_counts;
    int u_stride, c_stride;
};

// One sorted array per step and what to derive from it.  Real items (value < n_real) are the
// gradient contributions; every distinct key must also hold at least one other item (its
// zero-gradient member of the update set), which the stable sort leaves behind the real ones.
// Rows with at most `direct_max` real items get no chunks (their consumer sums
// the items itself); longer rows are cut into chunks of `chunk` items.
struct SegJob {
    const uint32_t* keys;  // [n_seg, N] sorted
    const uint32_t* vals;
    int N, n_real, chunk, direct_max;
    SegPlan plan;
};
// j1 (or null): a second job with the same number of segments, served by the same launches.
// scratch: find_segments_scratch_words(j0.N, j1 ? j1->N : 0, n_seg) words, no initial content needed.
size_t find_segments_scratch_words(int N0, int N1, int n_seg);
void launch_find_segments2(const SegJob& j0, const SegJob* j1, int n_seg, uint32_t* scratch, hipStream_t stream);

// ---- step phase ----------------------------------------------------------

struct ScoreShape {
    int S, B, T, Dp;   // Dp: embedding size rounded up to a multiple of 4
    int score_fn, dist_fn, loss_fn;
    float gamma, loss_scale;
    float softmax_correction;      // already multiplied by the correction weight
    float negative_adversarial_scale;
    int use_mfma;                  // L2 / dot scoring on the matrix cores (else the VALU kernels)
    int operands_dense;            // a-operand rows already hold the predicted tails (launch_gather_operands)
    // merged tails (launch_merge_tails), or null: block d scores its first tcount[d] tail columns
    // only (in whole groups of `tpad` columns, never more than T), column j standing for
    // tmult[d * T + j] tail positions: one of them the label's if the positive's label names the
    // column, the others negatives
    // (default member initialisers: a shape built field by field scores every column)
    const uint32_t* tcount = nullptr;
    const float* tmult = nullptr;
    int tpad = 64;
};
// the tail columns block d scores and differentiates
__host__ __device__ inline int tail_limit(const uint32_t* tcount, int d, int T, int tpad) {
    if (!tcount) return T;
    const int t = ((int)tcount[d] + tpad - 1) / tpad * tpad;
    return t < T ? t : T;
}

// Dense float32 operand matrix [n_rows, Dp] from indexed rows: rows [0, n_head)
// combined with their relation row (rel_mode 1 add, 2 multiply, 3 complex product on the
// halves [0, half) | [half, 2 half) of the row, 4 rotation by the row's `half` phases).
// With `out16` the values are rounded to bfloat16, stored there, and the float32
// copy holds the same rounded values.
// `tail_cols` (or null): rows from n_head on are the blocks' tail columns [S, T]; the columns past a
// block's limit (tail_limit) are left alone.
struct TailCols {
    const uint32_t* tcount = nullptr;
    int T = 1, tpad = 1;
    // whether the row `t` places behind the heads is to be gathered
    __device__ bool live(int t) const {
        if (!tcount || t < 0) return true;
        const int d = t / T;
        return t - d * T < tail_limit(tcount, d, T, tpad);
    }
};
void launch_gather_operands(const RowSource& ent, const float* rel, const uint32_t* crel, int rel_mode,
                            int half, int n_head, int n_rows, int Dp, float* out, uint16_t* out16,
                            hipStream_t stream, const TailCols* tail_cols = nullptr);

// Batched bfloat16 product on the matrix cores: C[z] = A[z] . Bt[z]^T, float32 out.
// Strides in elements.  Optional rows added to the output: output row m gets row
// add_index[m] of add_base (row 0 for m >= *add_count), columns as C's.
struct GemmNT {
    const uint16_t* A;  int64_t lda, a_batch;   // [M, K], or [K, M] with a_kmajor
    const uint16_t* Bt; int64_t ldb, b_batch;   // [N, K], or [K, N] with b_kmajor
    float* C;           int64_t ldc, c_batch;   // [M, N]
    int M, N, K, batches;
    float* part; int ksplit;                    // scratch for split contractions (or null); set by the launcher
    const char* add_base; int64_t add_pitch; int add_etype;
    const uint32_t* add_index; const uint32_t* add_count;
    // device-side counts (or null), one per batch limit_stride words apart (0: one for all):
    // output rows from the m_limit on and output columns from the n_limit on are not computed
    // (whole tiles: a tile that starts below the limit is computed in full); contraction columns
    // from the k_limit (rounded up to the slab) on are taken as zero
    const uint32_t* m_limit; const uint32_t* k_limit; const uint32_t* n_limit;
    int limit_stride;
    // the operand lies with the contraction index outermost (even pitch, 4-byte aligned base);
    // b_kmajor = 2: and Bt points to float32 values (pitch and batch stride in floats, 8-byte
    // aligned base), rounded to bfloat16 while staged
    int a_kmajor, b_kmajor;
};
bool gemm_nt_bf16_ok(int M, int N, int K);
int gemm_nt_bf16_ksplit(int M, int N, int K, int batches);  // partials needed: batches * ksplit * M * N floats
void launch_gemm_nt_bf16(const GemmNT& g, hipStream_t stream);
// Scores of every block: a-operand row (d,b) = entity row of contribution
// d*B+b combined with relation crel[d*B+b]; b-operand row (d,t) = entity row of
// contribution S*B + d*T + t.  With `fused_loss` the logsigmoid loss and the
// backward coefficient are produced in the epilogue; otherwise the raw score is
// stored in `coef` (and the L2 distance in `dist`) for launch_loss_rows.
// loss_part receives S * n_part partial sums (n_part = tiles per block).
void launch_score_fwd(const ScoreShape& sh, const RowSource& ent, const float* rel,
                      const uint32_t* crel, const uint32_t* clabel, float* coef, float* dist,
                      uint32_t* nearflag, float* loss_part, bool fused_loss, hipStream_t stream);
// raw scores of rows `a` against rows `b` of a second source (no relation, no loss): out [S, B, T]
void launch_score_fwd_rows(const ScoreShape& sh, const RowSource& a, const RowSource& b, float* scores,
                           hipStream_t stream);
// words of the near-identical-pair flag matrix the L2 matrix-core path needs
inline size_t nearflag_words(const ScoreShape& sh) {
    return (size_t)sh.S * ((sh.B + 31) / 32) * ((sh.T + 31) / 32);
}
int score_fwd_parts(const ScoreShape& sh);

// Row-wise losses (softmax; logsigmoid with adversarial weighting): converts
// the raw scores in `coef` to backward coefficients in place; loss_part gets
// S * B partial sums.  `coef16` (may be null): a bfloat16 copy of the coefficients; with
// `keep_f32` false and the softmax row held in registers only that copy is written.
void launch_loss_rows(const ScoreShape& sh, const uint32_t* clabel, float* coef, const float* dist,
                      float* loss_part, uint16_t* coef16, hipStream_t stream, bool keep_f32 = true);

// Stand-alone loss ops.  log_sigmoid: y = logsigmoid(x), dx = dy * its derivative (dy null: 1);
// form 0 evaluates them as launch_loss_rows does, form 1 as the fused scoring epilogue does.
// log_softmax: rows of `cols`; with dy null out = log_softmax(x), otherwise `x` holds the
// forward's output and out = dy - exp(x) * sum(dy).
void launch_log_sigmoid(const float* x, const float* dy, float* y, float* dx, int64_t n, int form,
                        hipStream_t stream);
void launch_log_softmax(const float* x, const float* dy, float* out, int64_t rows, int64_t cols,
                        hipStream_t stream);

// Gradient rows of every contribution: grad[c, :] for head contributions
// (w.r.t. the predicted tail / the head-times-relation product) and tail
// contributions, from the coefficient matrix.
void launch_score_bwd(const ScoreShape& sh, const RowSource& ent, const float* rel,
                      const uint32_t* crel, const float* coef, const uint32_t* nearflag, float* grad,
                      hipStream_t stream);

// Where gradient contributions come from.  transform: 0 none; 1 multiply head
// rows (c < n_head) by rel[crel[c]] (DistMult, entity plan); 2 multiply by the
// head entity row (DistMult, relation plan); 3 / 4 the same two for ComplEx: the
// product with the complex conjugate on the halves [0, half) | [half, 2 half); 5 / 6 for
// RotatE: the rotation back (entity plan), the phases' gradient in float16 (relation plan).
struct ContribSrc {
    const uint32_t* sorted_item;  // this step's sorted values
    const float* grad;            // [R, Dp]
    int transform, n_head, half;
    const float* rel;
    const uint32_t* crel;
    RowSource ent;
};

// Deterministic segmented reduction, first level (rows with many
// contributions only): one workgroup per chunk sums the chunk's gradient rows
// in a fixed order into partial[chunk, :].
struct ReduceArgs {
    ContribSrc src;
    const uint32_t* chunk_pos;
    const uint32_t* chunk_len;
    const uint32_t* counts;       // {rows, chunks}
    int max_chunks;
    int chunk;                    // most contributions a chunk holds
    float* partial;               // [max_chunks, Dp]
    int Dp;
};
void launch_reduce_chunks(const ReduceArgs& a, hipStream_t stream);
void launch_reduce_chunks2(const ReduceArgs& a0, const ReduceArgs& a1, hipStream_t stream);  // one launch

// Second level fused with Adam: one wave per distinct row sums its
// contributions (few: directly; many: its chunk partials) in order, applies the
// update in place and (optionally) stores the summed gradient.
struct AdamArgs {
    ContribSrc src;
    const uint32_t* uniq_key;
    const uint32_t* seg_start;
    const uint32_t* seg_real;
    const uint32_t* chunk_off;
    const uint32_t* counts;
    int max_rows;
    const float* partial;      // [chunks, Dp]
    const float* grad_direct;  // [rows, Dp] used instead of the contributions when non-null
    float* grad_out;           // [rows, Dp] or null
    char* p_base;              // parameter rows: p_base + key * pitch
    char* m_base;
    char* v_base;
    int64_t pitch;
    int p_etype, m_etype;      // ET_* of the parameter and of the two moments
    int Dp;
    int v_is_sqrt;
    int no_update;             // only form the summed gradient (grad_out), leave the rows alone
    const float* alpha;        // [n_alpha] step sizes
    uint32_t rows_per_alpha;   // alpha index = key / rows_per_alpha (0: always alpha[0])
    float beta_m, beta_v, one_minus_beta_m, one_minus_beta_v, epsilon, weight_decay;
    // norm regularisers (launch_reg_rows), or null: added to the row's gradient before the
    // update / to what grad_out receives
    const float* grad_add;      // [rows, Dp]
    const float* grad_out_add;  // [rows, Dp]
};
void launch_adam_rows(const AdamArgs& a, hipStream_t stream);
void launch_adam_rows2(const AdamArgs& a0, const AdamArgs& a1, hipStream_t stream);  // one launch
// The same two updates without the first-level reduction (launch_reduce_chunks) before them:
// a row with chunks ("hot", SegPlan::hot_rows) is summed and updated by workgroups of its own,
// one per 32 columns, the other rows by one wave each as in launch_adam_rows.  Contributions
// as stored (ContribSrc::transform 0) only.  max_hot: upper bound of *hot_count.
struct HotRows {
    const uint32_t* hot_rows;
    const uint32_t* hot_count;
    int max_hot;
    // or null / 0: the row of every chunk (SegPlan::chunk_row) and an upper bound of the step's
    // chunks: the launch then has one workgroup per chunk, and the first 1, 2, 4 or 8 of a row's
    // chunk workgroups share its columns
    const uint32_t* chunk_row = nullptr;
    int n_chunks = 0;
};
void launch_adam_rows_hot2(const AdamArgs& a0, const HotRows& h0, const AdamArgs& a1, const HotRows& h1,
                           hipStream_t stream);

// loss[s] = sum over steps and parts of loss_part / n_step, in a fixed order; `extra`
// (or null) holds one more term per (step, shard).
void launch_loss_finalize(const float* loss_part, int n_step, int S, int n_part, float scale,
                          float* loss, hipStream_t stream, const float* extra = nullptr,
                          float* step_sums = nullptr);

// Norm regularisers (src/poplar_kge.cpp:430-437, 463-465) on the distinct rows of one step:
// weight * (sum_k |x_k^power|)^(1/power) of the embedding, of feature . W (hidden - embedding)
// and of hidden, each counted twice per gathered slot (the reference evaluates them once
// for the heads and once for the tails, on the same gathered rows).  A row gathered by
// `mult` slots (segment members that are not gradient contributions) counts mult times.
struct RegArgs {
    const uint32_t* uniq_key; const uint32_t* seg_start; const uint32_t* seg_real; const uint32_t* counts;
    int max_rows;
    const char* emb_base; int64_t pitch; int emb_etype;
    const float* hidden;        // [rows, Dp] or null (no features: hidden = embedding)
    int D, Dp;
    float power[3], weight[3];  // embedding, feature product, hidden
    float loss_scale;
    float* add_val;             // [rows, Dp] gradient for the embedding
    float* add_fh;              // [rows, Dp] gradient for the feature product (or null)
    float* loss_row;            // [rows] the row's share of the loss
    float uses;                 // entityHidden calls this launch stands for: 2 (heads' and tails' calls
                                // see the same tensors) or 1 (one launch per call, with its hidden rows)
    int accumulate;             // add to add_val and loss_row instead of overwriting them
};
void launch_reg_rows(const RegArgs& a, hipStream_t stream);
// out[s] = sum of loss_row over the distinct rows owned by shard s (key / rows_per_shard), fixed order
void launch_reg_loss(const uint32_t* uniq_key, const uint32_t* counts, const float* loss_row,
                     uint32_t rows_per_shard, int S, float* out, hipStream_t stream);

// ---- feature projection (hidden = emb + feature * W) -----------------------
struct FeatureArgs {
    const uint32_t* uniq_key;
    const uint32_t* counts;
    int max_rows;
    const char* emb_base;   // table + emb offset; null: launch_hidden_fwd leaves the embedding out
    const char* feat_base;  // table + feature offset
    int64_t pitch;
    int emb_etype, feat_etype;
    int Dp, Fp;
    const float* proj;      // [Fp, Dp]
    float* featd;           // scratch [max_rows, Fp]: the distinct rows' features, float32
    float* gproj_part;      // scratch [16, Fp, Dp]: split-contraction partials of the projection gradient
    int use_mfma;
    // bfloat16 products (null without bfloat16 scoring): features [max_rows, Fp] and their
    // transpose, W^T [Dp, Fp], grad_rows^T [Dp, max_rows]
    uint16_t* feat16;
    int round_bf16;         // features and W enter their products rounded to bfloat16
    float* projR;           // scratch [Fp, Dp]: W rounded, for the float32 kernels
};
void launch_hidden_fwd(const FeatureArgs& a, float* hidden, hipStream_t stream);
// gproj[f, :] = sum_u feature[u, f] * grad_rows[u, :]
void launch_proj_grad(const FeatureArgs& a, const float* grad_rows, float* gproj,
                      hipStream_t stream);

// ---- predict -----------------------------------------------------------------
// Merge scores[q, 0..n_valid) (indices first_index + column) into each query's
// n_best best (score descending, index ascending; n_best <= 1024).
void launch_topk_merge(const float* scores, int64_t ld, int n_queries, int n_valid, uint32_t first_index,
                       int n_best, float* best_score, uint32_t* best_index, hipStream_t stream);
void launch_row_range(uint32_t base, int n_live, int n, uint32_t* out, hipStream_t stream);

// ---- table access ----------------------------------------------------------
void launch_rows_gather(const void* buf, const uint32_t* idx, void* out, int64_t n,
                        int64_t row_bytes, hipStream_t stream);
void launch_rows_scatter(void* buf, const uint32_t* idx, const void* data, int64_t n,
                         int64_t row_bytes, hipStream_t stream);

struct RowLayout {
    int D, F, Dp, Fp;
    int emb_etype, mom_etype, feat_etype;
    int64_t off_m, off_s, off_f, pitch;  // bytes; embedding at offset 0
};
// logical float32 rows [n, 3D+F] <-> physical rows at base + idx[i]*pitch
void launch_rows_to_logical(const RowLayout& L, const char* base, const uint64_t* rows, int64_t n,
                            float* out, hipStream_t stream);
void launch_rows_from_logical(const RowLayout& L, char* base, const uint64_t* rows, int64_t n,
                              const float* in, hipStream_t stream);
// write_entity: embedding ~ N(0, sigma) from a counter-based generator keyed by
// (seed, row, column); zero moments; features from `features` [n, F] float32.
void launch_init_rows(const RowLayout& L, char* base, const uint64_t* rows, int64_t n,
                      const float* features, float sigma, uint32_t seed, hipStream_t stream);

// ---- standalone ops --------------------------------------------------------
void launch_distance(int dist_fn, const float* a, const float* b, float* out, int M, int N, int D,
                     hipStream_t stream);
void launch_distance_grad(int dist_fn, const float* a, const float* b, const float* dist,
                          const float* g, float* grad, int M, int N, int D, hipStream_t stream);
void launch_adam_flat(float* p, float* m, float* v, const float* g, int64_t n, float alpha,
                      float beta_m, float beta_v, float epsilon, float weight_decay, int v_is_sqrt,
                      hipStream_t stream);
void launch_fill_u32(uint32_t* p, uint32_t value, int64_t n, hipStream_t stream);
void launch_iota_keys(const uint32_t* idx, uint32_t* keys, uint32_t* vals, int64_t n, int64_t rows,
                      hipStream_t stream);
void launch_sum_partials_rows(const uint32_t* chunk_off, const float* partial, int64_t rows,
                              int64_t cols, float* out, hipStream_t stream);

// ---- TransH (src/poplar_kge.cpp:539-565) ----
// Operand matrices, dense float32 [R, Dp]: `pt` rows [0, S*B) predicted tails and rows [S*B, R)
// tails; `nt` rows [0, S*B) the positives' unit hyperplane normals and the same tails after
// them.  The relation table holds the raw normals as rows [n_rel, 2 n_rel).
// Heads of `pt` hold the gathered head rows on entry.
void launch_transh_predict(const float* rel, const uint32_t* crel, int n_rel, int n_head, int Dp, float* pt,
                           float* nt, hipStream_t stream);
struct TranshFwd {
    ScoreShape sh;
    const float* pt; const float* nt;
    const float* cmat;       // [S, B, T] c = n . tail (the dot-product forward on `nt`)
    const uint32_t* clabel;
    float* coef;             // [S, B, T] coefficient d loss / d distance (fused loss) or raw score
    float* dcm;              // [S, B, T] d loss / d c (fused loss) or q = sum_k sign(e) n; or null
    float* loss_part;        // as launch_score_fwd's, one part per 64 x 64 tile
};
void launch_transh_fwd(const TranshFwd& p, bool fused_loss, hipStream_t stream);
void launch_mul_rows(float* a, const float* b, int64_t n, hipStream_t stream);  // a[i] *= b[i]
struct TranshBwd {
    const float* pt; const float* nt;
    const float* coef; const float* cmat;  // [S, B, T]
    float* mm;    // [R, Dp] in: the dot-product backward on `nt` with coefficient dcm;
                  // out rows [0, S*B): d loss / d n complete
    float* grad;  // [R, Dp] out: d loss / d p (heads), d loss / d tail (tails)
    int S, B, T, Dp;
};
void launch_transh_bwd(const TranshBwd& p, hipStream_t stream);
// heads of `grad` -> the head rows' gradient; relgrad [2 n_head, Dp]: rows [0, n_head) the relation
// embedding rows' contributions, rows [n_head, 2 n_head) the normal rows'
void launch_transh_back(const RowSource& ent, const float* rel, const uint32_t* crel, int n_rel, int n_head,
                        int Dp, float* grad, const float* mm, float* relgrad, hipStream_t stream);

// ---- feature MLP (src/poplar_kge.cpp:453-458) ----
// hidden = value + relu([value | feature . W] . Up) . Down per distinct row
struct MlpArgs {
    const uint32_t* uniq_key; const uint32_t* counts; int max_rows;
    const char* emb_base; int64_t pitch; int emb_etype;
    int Dp, M;
    const float* up;    // [2 Dp, M]: rows [0, Dp) the embedding's, [Dp, 2 Dp) the projected features'
    const float* down;  // [M, Dp]
    float* concat;      // [max_rows, 2 Dp] the MLP's input (written by the forward)
    float* pre;         // [max_rows, M] pre-activations (written by the forward)
    int add_value;      // the forward's output: 1 value + MLP output (hidden), 0 the MLP output alone
};
// fproj [max_rows, Dp] = feature . W (launch_hidden_fwd with a null emb_base)
void launch_mlp_fwd(const MlpArgs& a, const float* fproj, float* hidden, hipStream_t stream);
void launch_mlp_bwd_rows(const MlpArgs& a, const float* g, const float* val_add, float* gpre, float* gval,
                         float* gfproj, hipStream_t stream);
// C [Ka, N] = f(A [rows, Ka])^T . B [rows, N] over the first *count rows, summed in row order
void launch_rows_atb(const float* A, int lda, int Ka, bool relu, const float* B, int ldb, int N,
                     const uint32_t* count, float* C, hipStream_t stream);

// ---- feature dropout (src/poplar_kge.cpp:459-461; src/pag/pag.cpp:596-617) ----
struct DropoutArgs {
    const uint32_t* uniq_key; const uint32_t* counts; int max_rows;
    const char* emb_base; int64_t pitch; int emb_etype;
    int Dp;
    uint32_t seed, step;   // model.seed, the optimiser step the mask belongs to
    uint32_t threshold;    // p * 2^32: an element is kept where its hash is at least this
    float scale;           // 1 / (1 - p)
    int enabled;           // 0: no dropout (separate feature networks alone): keep everything, scale 1
};
// hidden [2 max_rows, Dp]: row u = value + dropped feature part for the head use, row
// max_rows + u for the tail use; fh_head / fh_tail [max_rows, Dp] = the feature part for either
// use (one array unless the feature networks are separate)
void launch_dropout_hidden(const DropoutArgs& a, const float* fh_head, const float* fh_tail, float* hidden,
                           hipStream_t stream);
// out[c] = item_row[c] (+ n for c >= n_head): the hidden row contribution c reads
void launch_role_index(const uint32_t* item_row, int n_head, int n, uint32_t* out, hipStream_t stream);
// The feature part's gradient of every distinct row [max_rows, Dp] from its contributions:
// out_head alone (the head and tail uses added up) or one array per use
void launch_role_sums(const DropoutArgs& a, const ContribSrc& cs, const uint32_t* seg_start, const uint32_t* seg_real,
                      const float* fh_head, const float* fh_tail, const float* add_head, const float* add_tail,
                      float* out_head, float* out_tail, hipStream_t stream);  // add_*: null, or rows added per use

}  // namespace kge
