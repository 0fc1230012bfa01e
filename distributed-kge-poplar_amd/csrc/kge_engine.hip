// Host side of libkge_hip.so: settings, validation, command dispatch and the
// step schedule behind the C-ABI of include/kge_hip.h.
//
// Mirrors, for the training path only, poplar_kge::Engine
// (src/poplar_kge.cpp:914-1006): Model settings (:198-286), stream validation
// (GetData, :69-106), the commands of EngineImpl::run (:950-998) and the order
// of operations of Model::trainStep (:664-707) / trainStepLoop (:709-741).
#include "../../include/kge_hip.h"
#include "kge_kernels.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <memory>
#include <condition_variable>
#include <exception>
#include <mutex>
#include <thread>
#include <sstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

using namespace kge;

namespace {

#define HIP_CHECK(expr)                                                                      \
    do {                                                                                     \
        hipError_t e_ = (expr);                                                              \
        if (e_ != hipSuccess) {                                                              \
            std::ostringstream m_;                                                           \
            m_ << "HIP error " << hipGetErrorString(e_) << " at " << __FILE__ << ":" << __LINE__ \
               << " (" #expr ")";                                                            \
            throw std::runtime_error(m_.str());                                              \
        }                                                                                    \
    } while (0)

const char* kind_name(int kind) {
    switch (kind) {
        case KGE_STR: return "string";
        case KGE_F32: return "float";
        case KGE_U32: return "unsigned int";
        case KGE_F16: return "half";
        case KGE_BOOL: return "bool";
        case KGE_FLOAT: return "float (scalar)";
        case KGE_UINT: return "unsigned (scalar)";
        case KGE_MAP: return "map";
    }
    return "<unknown>";
}

std::string shape_str(const size_t* shape, size_t rank) {
    std::ostringstream s;
    s << "(";
    for (size_t i = 0; i < rank; ++i) s << (i ? ", " : "") << shape[i];
    s << ")";
    return s.str();
}
std::string shape_str(const std::vector<size_t>& v) { return shape_str(v.data(), v.size()); }

// The reference's get/extract helpers (src/poplar_kge.cpp:38-67).
struct Items {
    const kge_item* items;
    size_t n;
    const kge_item* find(const std::string& key) const {
        for (size_t i = 0; i < n; ++i)
            if (items[i].key && key == items[i].key) return &items[i];
        return nullptr;
    }
    const kge_item& get(const std::string& key) const {
        const kge_item* it = find(key);
        if (!it) throw std::invalid_argument("Key not found '" + key + "'");
        return *it;
    }
    const kge_item& typed(const std::string& key, int kind) const {
        const kge_item& it = get(key);
        if (it.kind != kind) {
            std::ostringstream msg;
            msg << "Key '" << key << "' holds value of unexpected type. Expected: '" << kind_name(kind)
                << "', actual: '" << kind_name(it.kind) << "'.";
            throw std::invalid_argument(msg.str());
        }
        return it;
    }
    unsigned uint(const std::string& key) const { return (unsigned)typed(key, KGE_UINT).num; }
    float flt(const std::string& key) const { return (float)typed(key, KGE_FLOAT).num; }
    bool boolean(const std::string& key) const { return typed(key, KGE_BOOL).num != 0; }
    std::string str(const std::string& key) const { return typed(key, KGE_STR).str; }
    // stream binding with strict dtype and shape checks (GetData, :69-106)
    void* array(const std::string& name, int kind, const std::vector<size_t>& shape) const {
        const kge_item& it = get(name);
        if (it.kind != KGE_F32 && it.kind != KGE_U32 && it.kind != KGE_F16) {
            std::ostringstream msg;
            msg << "'" << name << "' expected type " << kind_name(kind) << ", actual: <not found> ("
                << kind_name(it.kind) << ")";
            throw std::invalid_argument(msg.str());
        }
        if (it.kind != kind) {
            std::ostringstream msg;
            msg << "'" << name << "' expected array of type " << kind_name(kind)
                << ", actual: " << kind_name(it.kind);
            throw std::invalid_argument(msg.str());
        }
        if (it.rank != shape.size() || !std::equal(shape.begin(), shape.end(), it.shape)) {
            std::ostringstream msg;
            msg << "'" << name << "' expected array of shape " << shape_str(shape)
                << ", actual: " << shape_str(it.shape, it.rank);
            throw std::invalid_argument(msg.str());
        }
        return it.data;
    }
};

template <class T>
struct DevBuf {
    T* p = nullptr;
    size_t n = 0;
    void alloc(size_t count) {
        release();
        n = count;
        if (count) HIP_CHECK(hipMalloc((void**)&p, count * sizeof(T)));
    }
    void zero(hipStream_t s) {
        if (n) HIP_CHECK(hipMemsetAsync(p, 0, n * sizeof(T), s));
    }
    void release() {
        if (p) (void)hipFree(p);
        p = nullptr;
        n = 0;
    }
    ~DevBuf() { release(); }
};

int round_up(int x, int m) { return (x + m - 1) / m * m; }
int elem_size(int et) { return et == ET_F32 ? 4 : 2; }
int bit_length(uint64_t x) { int b = 0; while (x) { ++b; x >>= 1; } return b; }

float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ff, u;
    if (exp == 0) {
        if (man == 0) u = sign;
        else {
            int e = -1;
            do { ++e; man <<= 1; } while (!(man & 0x400));
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ff) << 13);
        }
    } else if (exp == 31) u = sign | 0x7f800000u | (man << 13);
    else u = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
uint16_t float_to_half(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000;
    uint32_t mag = u & 0x7fffffffu;
    if (mag >= 0x7f800000u) return (uint16_t)(sign | 0x7c00 | (mag > 0x7f800000u ? 0x200 : 0));
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00);
    if (mag < 0x38800000u) {  // subnormal half
        if (mag < 0x33000000u) return (uint16_t)sign;
        const int e = (int)(mag >> 23);
        uint32_t man = (mag & 0x7fffffu) | 0x800000u;
        const int shift = 126 - e;  // total right shift: 13 + (113 - e)
        const uint32_t half = 1u << (shift - 1), rem = man & ((1u << shift) - 1);
        man >>= shift;
        if (rem > half || (rem == half && (man & 1))) ++man;
        return (uint16_t)(sign | man);
    }
    mag += 0xfffu + ((mag >> 13) & 1u);
    return (uint16_t)(sign | ((mag - 0x38000000u) >> 13));
}

enum KernelId {
    K_PLAN = 0, K_HIDDEN, K_GATHER, K_FWD, K_LOSS, K_BWD, K_REDUCE_ENT, K_ADAM_ENT, K_REDUCE_REL, K_ADAM_REL,
    K_PROJ_GRAD, K_ADAM_PROJ, K_COUNT
};

struct Variable {
    std::string name;
    std::vector<size_t> shape;
};

}  // namespace

struct kge_engine {
    // ---- settings (src/poplar_kge.cpp:198-236) ----
    int S, n_entity, n_rel, D, F, B, A, T, NR, R;
    // TransH keeps a second row per relation, the hyperplane normal (relation_normal), as rows
    // [n_rel, 2 n_rel) of the relation table: rel_copies = 2, n_rel_rows = 2 n_rel
    int rel_copies = 1, n_rel_rows = 0;
    // model.share_feature_networks = false: a head and a tail feature network (src/poplar_kge.cpp:268-273);
    // every parameter / gradient buffer of the feature path then holds the head's part and
    // the tail's part one after the other, and a distinct row has a hidden row per role
    int nets = 1;
    float dropout = 0.f;  // model.feature_dropout (training only): two hidden rows per distinct row
    DevBuf<float> fh;          // the feature part of hidden, before dropout
    DevBuf<uint32_t> role_idx;  // the hidden row of every contribution
    int step_of_first = 0;     // optimiser step of the first step of the running call
    // {distinct rows, chunks} of the entity plan and of the relation plan for every step of the
    // resident batch, read back once after the plan phase of a call with enough steps to pay
    // for the wait: the per-row and per-chunk launches then start no workgroup that only finds
    // out it has nothing to do (two thirds of them under power-law sampling)
    // (pinned host memory: the copies are asynchronous and waited for only when the first launch
    // that needs them is due, behind the first step's gather and scoring launches)
    // per step {distinct rows, chunks, rows with chunks, contributions of the biggest row}, which
    // the segment kernel writes straight into this (device-visible) host memory
    uint32_t *h_e_counts = nullptr, *h_r_counts = nullptr;  // [n_step][4] each
    uint32_t *d_e_counts = nullptr, *d_r_counts = nullptr;  // the same memory as the device addresses it
    void* h_pin = nullptr;          // the two arrays above, the step sizes and the loss
    float* h_alpha_pin = nullptr;
    float* h_loss_pin = nullptr;
    float* d_loss_pin = nullptr;  // the device's view of h_loss_pin: the loss kernel stores there, no copy follows
    hipEvent_t counts_ready = nullptr;
    hipEvent_t counts_wait = nullptr;  // the event the host waits for before it reads the counts
    bool counts_pending = false;
    bool counts_known = false;
    int plan_readback_steps = 8;  // additive setting execution.plan_readback_steps: calls of at least this many steps
    int mlp = 0;  // model.feature_mlp_size: hidden = value + relu([value | feature . W] . Up) . Down
    int score_fn, dist_fn, loss_fn;
    bool shared_table;
    float gamma, init_scale, beta_m, beta_v, epsilon, weight_decay, loss_scale, softmax_cw, neg_adv;
    float lr_mod_entity = 1.f, lr_mod_rel = 1.f, lr_mod_normal = 1.f;
    float lr_mod_proj[2] = {1.f, 1.f}, lr_mod_up[2] = {1.f, 1.f}, lr_mod_down[2] = {1.f, 1.f};  // per network
    uint32_t seed;
    int n_step, rw_batch;
    int predict_hr_batch = 0, predict_n_best = 0;
    int predict_chunk_rows = 0;  // additive setting execution.predict_chunk_rows: tails scored per launch (0: chosen from the number of queries)
    int stream_kind;  // KGE_F32 or KGE_F16: dtype of the entity read/write streams
    bool profile_kernels = false;
    // additive setting execution.scoring: "mfma_bf16x3" (2, the default: matrix cores, the forward
    // products from six bfloat16 instructions on three-piece float32 operands where shapes are
    // aligned), "mfma" (1: float32 matrix instructions only), "valu" (0)
    int use_mfma = 2;
    bool score_bf16 = false;  // additive setting execution.scoring_dtype = "float32" | "bfloat16"
    int chunk = 64;       // contributions per first-level chunk (rows with many contributions; 256 measured no faster)
    int direct_max = 16;  // rows with at most this many contributions are summed by their Adam wave

    RowLayout L;
    int64_t n_rows;
    int Dp, Fp;
    std::vector<Variable> variables;

    // ---- device state ----
    hipStream_t stream = nullptr;
    // predict: the n_best merge of one chunk of tails runs here while the next chunk is gathered
    // and scored on `stream` (the merge occupies one workgroup per query, a fraction of the chip)
    hipStream_t merge_stream = nullptr;
    static constexpr int kScoreBuffers = 3;  // a sweep's first merge (list still filling) takes three chunks' time
    hipEvent_t scored[kScoreBuffers] = {}, merged[kScoreBuffers] = {};
    // pinned staging for a predict run's queries and results (pageable copies cost ~50 us each)
    void* p_pin = nullptr;
    size_t p_pin_bytes = 0;
    DevBuf<char> table;
    DevBuf<float> rel, rel_m, rel_v, proj, proj_m, proj_v;
    uint32_t step = 0;

    // staged batch
    // The batch on the device, step by step: step i's remote [S, NR], a2a [S, S, A], head, relation,
    // tail [S, B] back to back (idx_words words per step), so that any range of steps is one
    // contiguous upload.  h_idx: the same layout in pinned host memory, filled (and every index
    // checked) by the host while it re-orders the caller's [S, n_step, ...] arrays.
    DevBuf<uint32_t> d_idx;
    uint32_t* h_idx = nullptr;
    size_t idx_words = 0, off_a2a = 0, off_head = 0, off_relation = 0, off_tail = 0;
    // Host arrays are taken in chunks of steps: while the device runs one chunk, the host checks
    // and re-orders the next, whose upload (copy_stream) and plan (plan_stream) run beside the
    // current chunk's kernels
    hipStream_t copy_stream = nullptr, plan_stream = nullptr;
    std::vector<hipEvent_t> chunk_copied, chunk_planned;
    bool staged = false;
    // plan
    DevBuf<uint32_t> ckey, crel, clabel, ek_a, ev_a, ek_b, ev_b, rk_a, rv_a, rk_b, rv_b, hist, seg_scratch;
    DevBuf<uint32_t> e_uniq, e_seg, e_coff, e_cpos, e_clen, e_counts, e_item_row, e_real;
    DevBuf<uint32_t> r_uniq, r_seg, r_coff, r_cpos, r_clen, r_counts, r_real;
    DevBuf<uint32_t> e_hot, e_hot_count, r_hot, r_hot_count;  // the rows with chunks, per step
    DevBuf<uint32_t> e_crow, r_crow;                          // the row of every chunk, per step
    DevBuf<uint32_t> nearflag;
    // additive setting execution.merge_tails (default true): a block scores one column per distinct
    // tail row, weighted by how many of its tail positions hold that row
    bool merge_tails = true;
    int tpad = 64;  // live tail columns come in whole groups of this many (the scoring kernels' tile)
    DevBuf<uint32_t> tkey, tcol, tcount;
    DevBuf<float> tmult;
    // additive setting execution.keep_gradients: the summed gradient of every distinct entity
    // row and of every relation row of the last step stays on the device for "grad_dump"
    bool keep_gradients = false;
    DevBuf<float> gkeep_e, gkeep_r;
    int last_step = -1;  // index (in the call's batch) of the step the kept gradients belong to
    int e_ustride, e_cstride, r_ustride, r_cstride, n_rel_items;
    uint32_t *e_sorted_vals = nullptr, *r_sorted_vals = nullptr;
    // step
    // predict scratch (allocated by the first predict call)
    DevBuf<uint32_t> p_idx, p_rel, p_count, p_best_i;
    DevBuf<float> p_opnd, p_scores, p_best_s, p_hidden, p_featd, p_opnd_n, p_cmat;
    DevBuf<uint16_t> opnd16, coef16, feat16;  // bfloat16 scoring operands
    // norm regularisers (src/poplar_kge.cpp:430-437): per distinct row gradients and loss shares
    float reg_p[3] = {3.f, 3.f, 3.f}, reg_w[3] = {0.f, 0.f, 0.f};
    bool reg_on = false;
    DevBuf<float> reg_val, reg_fh, reg_loss_row, reg_loss_part;
    // feature MLP: Up [2 Dp, M] and Down [M, Dp] with their moments and gradients; per distinct
    // row the projected features, the MLP's input, the pre-activations, their gradient, the
    // projected features' gradient and what the embedding's update must add
    DevBuf<float> up, up_m, up_v, down, down_m, down_v, g_up, g_down;
    DevBuf<float> mlp_fproj, mlp_concat, mlp_pre, mlp_gpre, mlp_gfp, mlp_gval, p_fproj, p_concat, p_pre;
    DevBuf<float> opnd_n, cmat, dcm, transh_mm, relgrad;  // TransH: [n | tails], c, d loss / d c, its products, relation contributions
    DevBuf<float> coef, dist, grad, opnd, partial, rel_partial, rel_gsum, hidden, gsum, gproj, featd, gproj_part, gemm_part, projR, loss_part, loss_step, d_alpha;
    // [n_step][entity, relation, normal, then per feature network projection, mlp up, mlp down][S]; the relation update indexes its two
    // groups as one array (key / rows_per_alpha), a shared table's [relation, normal] pair
    // sits in the first two entries of the relation group
    std::vector<float> h_alpha;
    int n_part;
    // io staging
    DevBuf<uint64_t> io_rows;
    DevBuf<float> io_data;
    DevBuf<uint32_t> io_idx;

    // timing
    hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr};
    float phase_ms[4] = {0, 0, 0, 0};  // upload, plan, steps, total of the last train_step_loop
    std::vector<hipEvent_t> kev;
    std::vector<int> kev_id;
    double kernel_ms[K_COUNT] = {0};
    uint32_t kernel_calls[K_COUNT] = {0};

    ~kge_engine() {
        for (auto& e : ev) if (e) (void)hipEventDestroy(e);
        for (auto& e : kev) (void)hipEventDestroy(e);
        if (p_pin) (void)hipHostFree(p_pin);
        if (h_pin) (void)hipHostFree(h_pin);
        if (counts_ready) (void)hipEventDestroy(counts_ready);
        for (auto& e : scored) if (e) (void)hipEventDestroy(e);
        for (auto& e : merged) if (e) (void)hipEventDestroy(e);
        if (merge_stream) (void)hipStreamDestroy(merge_stream);
        if (copy_stream) (void)hipStreamDestroy(copy_stream);
        if (plan_stream) (void)hipStreamDestroy(plan_stream);
        for (auto& e : chunk_copied) (void)hipEventDestroy(e);
        for (auto& e : chunk_planned) (void)hipEventDestroy(e);
        if (h_idx) (void)hipHostFree(h_idx);
        if (stream) (void)hipStreamDestroy(stream);
    }
};

namespace {

// zeroed rows behind the table's last: predict scores whole tiles of 64 consecutive rows in place
constexpr int64_t kSpareRows = 64;
// the most contributions a row may have for the update's launch to sum it (launch_adam_rows_hot2)
constexpr uint32_t kHotInUpdateMax = 4096;

// a step-size modifier of a feature network's parameter, by the variable's name
// (src/poplar_kge.cpp:321-327): [head_ | tail_]{feature_projection, mlp_up_projection, mlp_down_projection}
bool feature_modifier(kge_engine& E, const std::string& key, float value) {
    std::string name = key;
    int net = 0;
    if (E.nets == 2) {
        if (name.rfind("head_", 0) == 0) name = name.substr(5);
        else if (name.rfind("tail_", 0) == 0) { name = name.substr(5); net = 1; }
        else return false;
    }
    if (name == "feature_projection") E.lr_mod_proj[net] = value;
    else if (name == "mlp_up_projection" && E.mlp) E.lr_mod_up[net] = value;
    else if (name == "mlp_down_projection" && E.mlp) E.lr_mod_down[net] = value;
    else return false;
    return true;
}

// DistMult, ComplEx and RotatE form a row's gradient contributions from rows of the other
// table when they are summed (TransE's and TransH's are materialised before that)
bool contributions_read_tables(const kge_engine& E) {
    return E.score_fn == SCORE_DISTMULT || E.score_fn == SCORE_COMPLEX || E.score_fn == SCORE_ROTATE;
}

void parse_settings(kge_engine& E, const Items& s) {
    // the device: this library only drives a HIP device
    const std::string device = s.str("execution.device");
    if (device != "hip") {
        std::ostringstream msg;
        msg << "Unexpected setting \"device\": '" << device << "', expected \"hip\"";
        throw std::invalid_argument(msg.str());
    }
    E.seed = s.uint("model.seed");
    const std::string score = s.str("model.score_fn"), distance = s.str("model.distance_fn");
    E.S = (int)s.uint("model.n_shard");
    E.n_entity = (int)s.uint("model.n_entity");
    E.n_rel = (int)s.uint("model.n_relation_type");
    E.D = (int)s.uint("model.embedding_size");
    E.F = (int)s.uint("model.entity_feature_size");
    const unsigned mlp = s.uint("model.feature_mlp_size");
    const float dropout = s.flt("model.feature_dropout");
    const bool share = s.boolean("model.share_feature_networks");
    E.gamma = s.flt("model.gamma");
    E.init_scale = s.flt("model.init_scale");
    E.beta_m = s.flt("training.adam_beta_m");
    E.beta_v = s.flt("training.adam_beta_v");
    E.epsilon = s.flt("training.adam_epsilon");
    E.weight_decay = s.flt("training.weight_decay");
    const kge_item& mods = s.typed("training.learning_rate_modifiers", KGE_MAP);
    E.B = (int)s.uint("data.batch_size");
    E.A = (int)s.uint("data.a2a_size");
    E.neg_adv = s.flt("model.negative_adversarial_scale");
    const std::string loss = s.str("training.loss.type");
    const char* reg_names[3] = {"training.embedding_regularisation", "training.feature_regularisation",
                                "training.hidden_regularisation"};
    for (int i = 0; i < 3; ++i) {
        E.reg_p[i] = s.flt(std::string(reg_names[i]) + ".power");
        E.reg_w[i] = s.flt(std::string(reg_names[i]) + ".weight");
        if (E.reg_w[i] > 0) E.reg_on = true;
    }
    E.softmax_cw = loss == "softmax" ? s.flt("training.loss.correction_weight") : 0.f;
    E.loss_scale = s.flt("training.loss_scale");
    E.n_step = (int)s.uint("execution.train_steps_per_program_run");
    E.rw_batch = (int)s.uint("execution.rw_batch_size");
    E.predict_hr_batch = (int)s.uint("execution.predict_hr_batch_size");
    (void)s.uint("execution.predict_tail_batch_size");  // the device picks its own chunk of tails
    E.predict_n_best = (int)s.uint("execution.predict_n_best");

    // dtype of the entity table (src/poplar_kge.cpp:237-246) + additive layouts
    const std::string dtype = s.str("execution.dtype");
    int emb_et, mom_et, feat_et;
    if (dtype == "float32") { emb_et = mom_et = feat_et = ET_F32; E.stream_kind = KGE_F32; }
    else if (dtype == "float16") { emb_et = mom_et = feat_et = ET_F16; E.stream_kind = KGE_F16; }
    else {
        throw std::invalid_argument("'execution.dtype' must either be 'float16' or 'float32', not '" +
                                    dtype + "'");
    }
    auto parse_et = [&](const char* key, int& et) {
        if (!s.find(key)) return;
        const std::string v = s.str(key);
        if (v == "float32") et = ET_F32;
        else if (v == "float16") et = ET_F16;
        else if (v == "bfloat16") et = ET_BF16;
        else throw std::invalid_argument(std::string("'") + key + "' must be one of 'float32', 'float16', 'bfloat16', not '" + v + "'");
    };
    parse_et("execution.embedding_dtype", emb_et);
    parse_et("execution.feature_dtype", feat_et);
    E.shared_table = s.find("execution.shared_table") ? s.boolean("execution.shared_table") : false;
    if (E.reg_on && E.shared_table)
        throw std::invalid_argument("norm regularisers (weight > 0) need private shard tables: with "
                                    "'execution.shared_table' a row's loss share has no owning shard");
    E.profile_kernels = s.find("execution.profile_kernels") ? s.boolean("execution.profile_kernels") : false;
    if (s.find("execution.reduce_chunk")) {
        // the chunk tables are sized for chunks of at least 64 contributions (allocate: one chunk
        // per `chunk` contributions plus one per row that has more than direct_max)
        const unsigned v = s.uint("execution.reduce_chunk");
        if (v < 64 || v > 4096) throw std::invalid_argument("'execution.reduce_chunk' must be in [64, 4096]");
        E.chunk = (int)v;
    }
    if (s.find("execution.predict_chunk_rows")) {
        const unsigned v = s.uint("execution.predict_chunk_rows");
        if (v < 64 || v > (1u << 20)) throw std::invalid_argument("'execution.predict_chunk_rows' must be in [64, 1048576]");
        E.predict_chunk_rows = (int)v;
    }
    if (s.find("execution.plan_readback_steps")) E.plan_readback_steps = std::max(1, (int)s.uint("execution.plan_readback_steps"));
    if (s.find("execution.scoring")) {
        const std::string v = s.str("execution.scoring");
        if (v == "mfma") E.use_mfma = 1;
        else if (v == "mfma_bf16x3") E.use_mfma = 2;
        else if (v == "valu") E.use_mfma = 0;
        else throw std::invalid_argument("'execution.scoring' must be 'mfma', 'mfma_bf16x3' or 'valu', not '" + v + "'");
    }

    if (s.find("execution.scoring_dtype")) {
        const std::string v = s.str("execution.scoring_dtype");
        if (v == "bfloat16") E.score_bf16 = true;
        else if (v != "float32")
            throw std::invalid_argument("'execution.scoring_dtype' must be 'float32' or 'bfloat16', not '" + v + "'");
        if (E.score_bf16 && score != "DistMult")
            throw std::invalid_argument("'execution.scoring_dtype' = 'bfloat16' is implemented for "
                                        "'model.score_fn' = 'DistMult' (dot-product scores) only");
    }

    if (score == "TransE") E.score_fn = SCORE_TRANSE;
    else if (score == "DistMult") E.score_fn = SCORE_DISTMULT;
    else if (score == "ComplEx") E.score_fn = SCORE_COMPLEX;
    else if (score == "RotatE") E.score_fn = SCORE_ROTATE;
    else if (score == "TransH") E.score_fn = SCORE_TRANSH;
    else
        throw std::invalid_argument("'model.score_fn' must be one of 'TransE', 'ComplEx', 'RotatE', 'TransH', or "
                                    "'DistMult', not '" + score + "'");
    if (distance == "L1") E.dist_fn = DIST_L1;
    else if (distance == "L2") E.dist_fn = DIST_L2;
    else if (distance == "MatMul") E.dist_fn = DIST_DOT;
    else if (E.score_fn == SCORE_DISTMULT) E.dist_fn = DIST_DOT;
    else
        throw std::invalid_argument("'model.distance_fn' must be one of 'L1', 'L2' or 'MatMul', not '" +
                                    distance + "'");
    if (E.score_fn == SCORE_DISTMULT) E.dist_fn = DIST_DOT;  // distMultScore ignores the setting (:571-573)
    if (E.score_fn == SCORE_TRANSH) {  // so does transHScore: always the L1 norm (:563-564)
        E.dist_fn = DIST_L1;
        E.rel_copies = 2;
        if (E.score_bf16) throw std::invalid_argument("'execution.scoring_dtype' = 'bfloat16' is not implemented for TransH");
    }
    if ((E.score_fn == SCORE_COMPLEX || E.score_fn == SCORE_ROTATE) && E.D % 2)
        throw std::invalid_argument("'model.score_fn' = '" + score + "' needs an even 'model.embedding_size' "
                                    "(real and imaginary halves)");
    if (E.score_fn == SCORE_ROTATE && E.dist_fn == DIST_DOT)
        throw std::invalid_argument("'model.score_fn' = 'RotatE' scores by a distance: 'model.distance_fn' "
                                    "must be 'L1' or 'L2'");
    if (loss == "logsigmoid") E.loss_fn = LOSS_LOGSIGMOID;
    else if (loss == "softmax") E.loss_fn = LOSS_SOFTMAX;
    else
        throw std::invalid_argument("'training.loss.type' must be one of 'logsigmoid' or 'softmax', not '" +
                                    loss + "'");
    if (mlp > 0 && E.F == 0)
        throw std::invalid_argument("'model.feature_mlp_size' > 0 is implemented with entity features only "
                                    "('model.entity_feature_size' > 0)");
    if (mlp > 0 && E.score_bf16)
        throw std::invalid_argument("'model.feature_mlp_size' > 0 is not implemented together with "
                                    "'execution.scoring_dtype' = 'bfloat16'");
    E.mlp = (int)mlp;
    if (!(dropout >= 0.f && dropout < 1.f)) throw std::invalid_argument("'model.feature_dropout' must be in [0, 1)");
    E.dropout = E.F > 0 ? dropout : 0.f;  // without features the dropped tensor is all zeros
    if (E.dropout > 0 && E.score_bf16)
        throw std::invalid_argument("'model.feature_dropout' > 0 is not implemented together with "
                                    "'execution.scoring_dtype' = 'bfloat16'");

    E.nets = (!share && E.F > 0) ? 2 : 1;
    if (E.nets == 2 && E.score_bf16)
        throw std::invalid_argument("'model.share_feature_networks' = false is not implemented together with "
                                    "'execution.scoring_dtype' = 'bfloat16'");
    for (int i = 0; i < 3; ++i)
        if (E.reg_w[i] > 0 && !(E.reg_p[i] > 0))
            throw std::invalid_argument(std::string("'") + reg_names[i] + ".power' must be positive");
    if (E.S < 1 || E.B < 1 || E.A < 1 || E.D < 1 || E.n_entity < 1 || E.n_rel < 1 || E.n_step < 1 || E.rw_batch < 1)
        throw std::invalid_argument("sizes must be positive");
    if (E.S * E.A < 2) throw std::invalid_argument("n_shard * a2a_size must be at least 2");

    // parameter sharding check (addParameter, src/poplar_kge.cpp:294-300); a
    // shared table keeps every parameter whole, so nothing needs to divide
    if (!E.shared_table) {
        auto check = [&](const char* name, int dim0, int dim1) {
            if (dim0 % E.S) {
                std::ostringstream msg;
                msg << "Parameter '" << name << "' shape[0] (" << dim0 << ") is not divisible by n_shard ("
                    << E.S << "). Note shape: (" << dim0 << ", " << dim1 << ")";
                throw std::invalid_argument(msg.str());
            }
        };
        check("relation_embedding", E.n_rel, E.score_fn == SCORE_ROTATE ? E.D / 2 : E.D);
        check(E.nets == 2 ? "head_feature_projection" : "feature_projection", E.F, E.D);
        if (E.mlp) {
            check(E.nets == 2 ? "head_mlp_up_projection" : "mlp_up_projection", 2 * E.D, E.mlp);
            check(E.nets == 2 ? "head_mlp_down_projection" : "mlp_down_projection", E.mlp, E.D);
        }
    }
    E.n_rel_rows = E.n_rel * E.rel_copies;
    for (size_t i = 0; i < mods.map_len; ++i) {
        const std::string k = mods.map_keys[i];
        if (k == "entity_embedding") E.lr_mod_entity = mods.map_vals[i];
        else if (k == "relation_embedding") E.lr_mod_rel = mods.map_vals[i];
        else if (k == "relation_normal" && E.score_fn == SCORE_TRANSH) E.lr_mod_normal = mods.map_vals[i];
        else if (feature_modifier(E, k, mods.map_vals[i])) {}
        else
            throw std::invalid_argument("Bad training.learning_rate_modifier: unknown parameter '" + k + "'");
    }

    E.T = E.S * E.A;
    E.NR = E.B + E.T;
    E.R = E.S * E.NR;
    // additive: merged tails.  Not with TransH (its L1 part has kernels of its own) or the norm
    // regularisers (they count a row's members that carry no gradient as its gathered slots),
    // and for tail lists that fit one workgroup's sort.
    E.keep_gradients = s.find("execution.keep_gradients") ? s.boolean("execution.keep_gradients") : false;
    if (E.keep_gradients && (E.F || contributions_read_tables(E)))
        throw std::invalid_argument("'execution.keep_gradients' is implemented for score functions whose gradient "
                                    "contributions are used as stored (TransE, TransH) without entity features");
    E.merge_tails = s.find("execution.merge_tails") ? s.boolean("execution.merge_tails") : true;
    if (E.score_fn == SCORE_TRANSH || E.reg_on || E.T > kMergeMaxT) E.merge_tails = false;
    E.tpad = E.score_bf16 ? 128 : 64;  // the bfloat16 products work in tiles of 128
    E.Dp = round_up(E.D, (emb_et == ET_F32 && mom_et == ET_F32) ? 4 : 8);
    E.Fp = E.F ? round_up(E.F, feat_et == ET_F32 ? 4 : 8) : 0;
    RowLayout& L = E.L;
    L.D = E.D; L.F = E.F; L.Dp = E.Dp; L.Fp = E.Fp;
    L.emb_etype = emb_et; L.mom_etype = mom_et; L.feat_etype = feat_et;
    L.off_m = (int64_t)E.Dp * elem_size(emb_et);
    L.off_s = L.off_m + (int64_t)E.Dp * elem_size(mom_et);
    L.off_f = L.off_s + (int64_t)E.Dp * elem_size(mom_et);
    L.pitch = L.off_f + (int64_t)E.Fp * elem_size(feat_et);
    E.n_rows = E.shared_table ? (int64_t)E.n_entity : (int64_t)E.S * E.n_entity;
    if (E.n_rows >= ((int64_t)1 << (32 - kKeyFlagBits)))
        throw std::invalid_argument("the entity table must have fewer than 2^31 rows (32-bit sort keys: row number and one flag bit)");
    if (E.n_rows >= (int64_t)1 << 32) throw std::invalid_argument("more than 2^32 table rows");
    if ((int64_t)2 * E.R >= (int64_t)1 << 31) throw std::invalid_argument("batch too large");

    auto var = [&](const std::string& name, std::vector<size_t> shape) {
        E.variables.push_back({name, shape});
    };
    var("step", {(size_t)E.S});
    for (const char* suffix : {"", "/adam_m", "/adam_v"}) {
        // RotatE's rows are D / 2 phases (src/poplar_kge.cpp:248-249); the device rows keep the
        // full pitch, their upper half stays zero
        var(std::string("relation_embedding") + suffix,
            {(size_t)E.n_rel, (size_t)(E.score_fn == SCORE_ROTATE ? E.D / 2 : E.D)});
        if (E.score_fn == SCORE_TRANSH)  // :252-255
            var(std::string("relation_normal") + suffix, {(size_t)E.n_rel, (size_t)E.D});
        for (int net = 0; net < E.nets; ++net) {  // :256-273
            const std::string pre = E.nets == 2 ? (net ? "tail_" : "head_") : "";
            var(pre + "feature_projection" + suffix, {(size_t)E.F, (size_t)E.D});
            if (E.mlp) {
                var(pre + "mlp_up_projection" + suffix, {(size_t)(2 * E.D), (size_t)E.mlp});
                var(pre + "mlp_down_projection" + suffix, {(size_t)E.mlp, (size_t)E.D});
            }
        }
    }
}

void allocate(kge_engine& E) {
    int n_dev = 0;
    const hipError_t dev_err = hipGetDeviceCount(&n_dev);
    if (dev_err != hipSuccess || n_dev < 1) {
        (void)hipGetLastError();
        throw std::runtime_error(std::string("Could not attach to a HIP device (") +
                                 (dev_err != hipSuccess ? hipGetErrorString(dev_err) : "no device") + ")");
    }
    HIP_CHECK(hipStreamCreate(&E.stream));
    HIP_CHECK(hipStreamCreate(&E.merge_stream));
    for (auto& e : E.ev) HIP_CHECK(hipEventCreate(&e));
    for (auto& e : E.scored) HIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    for (auto& e : E.merged) HIP_CHECK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    const hipStream_t st = E.stream;

    E.table.alloc((size_t)(E.n_rows + kSpareRows) * E.L.pitch);
    E.table.zero(st);
    const size_t rel_n = (size_t)E.n_rel_rows * E.Dp, proj_n = (size_t)E.Fp * E.Dp;
    for (DevBuf<float>* b : {&E.rel, &E.rel_m, &E.rel_v}) { b->alloc(rel_n); b->zero(st); }
    for (DevBuf<float>* b : {&E.proj, &E.proj_m, &E.proj_v}) { b->alloc(E.nets * proj_n); b->zero(st); }

    const size_t ns = E.n_step, S = E.S, B = E.B, A = E.A, R = E.R, SB = S * B;
    E.off_a2a = R; E.off_head = E.off_a2a + S * S * A; E.off_relation = E.off_head + SB;
    E.off_tail = E.off_relation + SB; E.idx_words = E.off_tail + SB;
    E.d_idx.alloc(ns * E.idx_words);
    HIP_CHECK(hipHostMalloc((void**)&E.h_idx, ns * E.idx_words * 4, hipHostMallocDefault));
    HIP_CHECK(hipStreamCreate(&E.copy_stream));
    HIP_CHECK(hipStreamCreate(&E.plan_stream));

    E.ckey.alloc(ns * R);
    E.crel.alloc(ns * SB);
    E.clabel.alloc(ns * SB);
    for (DevBuf<uint32_t>* b : {&E.ek_a, &E.ev_a, &E.ek_b, &E.ev_b}) b->alloc(ns * 2 * R);
    E.n_rel_items = (int)((SB + E.n_rel) * E.rel_copies);
    for (DevBuf<uint32_t>* b : {&E.rk_a, &E.rv_a, &E.rk_b, &E.rv_b}) b->alloc(ns * E.n_rel_items);
    {   // the two sorts of a call run in shared launches: a histogram region each, both at the wider key's digit width
        const int bits = kKeyFlagBits + std::max(std::max(1, bit_length((uint64_t)E.n_rows - 1)), std::max(1, bit_length((uint64_t)E.n_rel_rows - 1)));
        E.hist.alloc(radix_sort_hist_words((int)(2 * R), (int)ns, bits) + radix_sort_hist_words(E.n_rel_items, (int)ns, bits));
    }
    E.seg_scratch.alloc(find_segments_scratch_words((int)(2 * R), E.n_rel_items, (int)ns));
    if (E.keep_gradients) {
        E.gkeep_e.alloc(R * E.Dp);
        E.gkeep_r.alloc((size_t)E.n_rel_rows * E.Dp);
    }
    if (E.merge_tails) {
        E.tkey.alloc(ns * S * E.T);
        E.tcol.alloc(ns * S * E.T);
        E.tmult.alloc(ns * S * E.T);
        E.tcount.alloc(ns * S);
    }
    {   // pinned host staging: plan counts [4][2 ns], step sizes [ns 9 S], loss [S]
        const size_t words = 8 * ns + ns * 9 * S + S;  // counts [2][ns][4]
        HIP_CHECK(hipHostMalloc(&E.h_pin, words * 4, hipHostMallocDefault));
        std::memset(E.h_pin, 0, words * 4);
        E.h_e_counts = (uint32_t*)E.h_pin; E.h_r_counts = E.h_e_counts + 4 * ns;
        E.h_alpha_pin = (float*)(E.h_r_counts + 4 * ns);
        void* dev_view = nullptr;
        HIP_CHECK(hipHostGetDevicePointer(&dev_view, E.h_pin, 0));
        E.d_e_counts = (uint32_t*)dev_view; E.d_r_counts = E.d_e_counts + 4 * ns;
        E.h_loss_pin = E.h_alpha_pin + ns * 9 * S;
        E.d_loss_pin = (float*)dev_view + (E.h_loss_pin - (float*)E.h_pin);
        HIP_CHECK(hipEventCreateWithFlags(&E.counts_ready, hipEventDisableTiming));
    }

    E.e_ustride = (int)R;
    // a row gets chunks only with more than direct_max contributions and then ceil(n / chunk) of
    // them: at most n / chunk + 1 per such row, of which there are at most R / (direct_max + 1)
    E.e_cstride = (int)(R / E.chunk + R / (E.direct_max + 1) + 2);
    E.e_real.alloc(ns * E.e_ustride);
    E.e_uniq.alloc(ns * E.e_ustride);
    E.e_seg.alloc(ns * (E.e_ustride + 1));
    E.e_coff.alloc(ns * (E.e_ustride + 1));
    E.e_cpos.alloc(ns * E.e_cstride);
    E.e_clen.alloc(ns * E.e_cstride);
    E.e_counts.alloc(ns * 2);
    E.e_hot.alloc(ns * E.e_cstride);
    E.e_crow.alloc(ns * E.e_cstride);
    E.e_hot_count.alloc(ns * 2);
    if (E.F) E.e_item_row.alloc(ns * R);
    E.r_ustride = E.n_rel_rows;
    E.r_cstride = (int)(SB * E.rel_copies / E.chunk + SB * E.rel_copies / (E.direct_max + 1) + 2);
    E.r_real.alloc(ns * E.r_ustride);
    E.r_uniq.alloc(ns * E.r_ustride);
    E.r_seg.alloc(ns * (E.r_ustride + 1));
    E.r_coff.alloc(ns * (E.r_ustride + 1));
    E.r_cpos.alloc(ns * E.r_cstride);
    E.r_clen.alloc(ns * E.r_cstride);
    E.r_counts.alloc(ns * 2);
    E.r_hot.alloc(ns * E.r_cstride);
    E.r_crow.alloc(ns * E.r_cstride);
    E.r_hot_count.alloc(ns * 2);

    E.coef.alloc(SB * E.T);
    const bool fused = E.loss_fn == LOSS_LOGSIGMOID && E.neg_adv <= 0.f && !E.score_bf16;
    if (!fused && E.dist_fn == DIST_L2) E.dist.alloc(SB * E.T);
    if (E.score_bf16) {
        E.opnd16.alloc(R * E.Dp);
        E.coef16.alloc(SB * E.T);
        // split-contraction partials of the two backward products
        const size_t p_head = (size_t)E.S * gemm_nt_bf16_ksplit(E.B, E.Dp, E.T, E.S) * E.B * E.Dp;
        const size_t p_tail = (size_t)E.S * gemm_nt_bf16_ksplit(E.T, E.Dp, E.B, E.S) * E.T * E.Dp;
        E.gemm_part.alloc(std::max(p_head, p_tail));
    }
    E.grad.alloc(R * E.Dp);
    E.opnd.alloc(R * E.Dp);
    if (E.merge_tails) {
        // columns past a block's distinct tails are never written; the kernels that read whole
        // tiles of them (and drop the results) must find finite values there
        E.opnd.zero(st);
        E.coef.zero(st);
        if (E.score_bf16) { E.opnd16.zero(st); E.coef16.zero(st); }
    }
    E.partial.alloc((size_t)E.e_cstride * E.Dp);
    E.rel_partial.alloc((size_t)E.r_cstride * E.Dp);
    if (contributions_read_tables(E)) E.rel_gsum.alloc((size_t)E.n_rel * E.Dp);
    if (E.score_fn == SCORE_TRANSH) {
        E.opnd_n.alloc(R * E.Dp);
        E.transh_mm.alloc(R * E.Dp);
        E.cmat.alloc(SB * E.T);
        E.dcm.alloc(SB * E.T);
        E.relgrad.alloc(2 * SB * E.Dp);
    }
    if (E.F) {
        const bool roles = E.dropout > 0 || E.nets == 2;
        E.hidden.alloc((roles ? 2 : 1) * R * E.Dp);
        if (E.dropout > 0) E.fh.alloc(E.nets * R * E.Dp);
        if (roles) E.role_idx.alloc(R);
        E.gsum.alloc(E.nets * R * E.Dp);
        E.gsum.zero(E.stream);  // rows past a step's distinct count are read (times zero): keep them finite
        E.featd.alloc(R * E.Fp);
        E.gproj_part.alloc((size_t)16 * E.Fp * E.Dp);
        if (E.score_bf16) {
            E.feat16.alloc(R * E.Fp);
            E.projR.alloc((size_t)E.Fp * E.Dp);
        }
        E.gproj.alloc(E.nets * proj_n);
        if (E.mlp) {
            const size_t M = E.mlp, up_n = 2 * (size_t)E.Dp * M, down_n = M * E.Dp, N = E.nets;
            for (DevBuf<float>* b : {&E.up, &E.up_m, &E.up_v, &E.g_up}) { b->alloc(N * up_n); b->zero(st); }
            for (DevBuf<float>* b : {&E.down, &E.down_m, &E.down_v, &E.g_down}) { b->alloc(N * down_n); b->zero(st); }
            E.mlp_fproj.alloc(N * R * E.Dp);
            E.mlp_concat.alloc(N * R * 2 * E.Dp);
            E.mlp_pre.alloc(N * R * M);
            E.mlp_gpre.alloc(N * R * M);
            E.mlp_gfp.alloc(N * R * E.Dp);
            E.mlp_gval.alloc(R * E.Dp);
            // rows past a step's distinct count are read by the projection gradient (times zero)
            E.mlp_gfp.zero(st);
        }
    }
    ScoreShape sh = {};
    sh.S = E.S; sh.B = E.B; sh.T = E.T;
    sh.score_fn = E.score_fn; sh.dist_fn = E.dist_fn; sh.use_mfma = E.use_mfma;
    E.n_part = fused ? score_fwd_parts(sh) : E.B;
    if (E.use_mfma && E.dist_fn == DIST_L2) {
        E.nearflag.alloc(nearflag_words(sh));
        E.nearflag.zero(st);
    }
    if (E.reg_on) {
        E.reg_val.alloc(R * E.Dp);
        if (E.F) E.reg_fh.alloc(((E.dropout > 0 || E.nets == 2) ? 2 : 1) * R * E.Dp);
        E.reg_loss_row.alloc(R);
        E.reg_loss_part.alloc(ns * S);
    }
    E.loss_part.alloc(ns * S * E.n_part);
    E.loss_step.alloc(ns * S);
    E.d_alpha.alloc(ns * 9 * S);

    const size_t io_n = (size_t)E.S * E.rw_batch;
    E.io_rows.alloc(io_n);
    E.io_idx.alloc(io_n);
    E.io_data.alloc(io_n * (3 * E.D + E.F));
    HIP_CHECK(hipStreamSynchronize(st));
}

// ---- variables: "read" / "write" (src/poplar_kge.cpp:977-991) ----------------

void run_read_write(kge_engine& E, bool write, const Items& in) {
    const std::string full_name = in.str("name");
    const Variable* var = nullptr;
    for (auto& v : E.variables) if (v.name == full_name) var = &v;
    if (!var) throw std::invalid_argument("Key not found '" + full_name + "'");
    if (full_name == "step") {
        uint32_t* v = (uint32_t*)in.array("value", KGE_U32, var->shape);
        if (write) E.step = v[0];
        else for (int s = 0; s < E.S; ++s) v[s] = E.step;
        return;
    }
    float* host = (float*)in.array("value", KGE_F32, var->shape);
    DevBuf<float>* buf = nullptr;
    size_t row0 = 0;  // first device row of the variable
    // the feature networks' variables: head_ / tail_ name the network when there are two
    std::string name = full_name;
    size_t net = 0;
    if (E.nets == 2 && (name.rfind("head_", 0) == 0 || name.rfind("tail_", 0) == 0)) {
        net = name[0] == 't';
        name = name.substr(5);
    }
    if (name == "relation_embedding") buf = &E.rel;
    else if (name == "relation_embedding/adam_m") buf = &E.rel_m;
    else if (name == "relation_embedding/adam_v") buf = &E.rel_v;
    else if (name == "relation_normal") { buf = &E.rel; row0 = E.n_rel; }
    else if (name == "relation_normal/adam_m") { buf = &E.rel_m; row0 = E.n_rel; }
    else if (name == "relation_normal/adam_v") { buf = &E.rel_v; row0 = E.n_rel; }
    else if (name == "feature_projection") { buf = &E.proj; row0 = net * E.Fp; }
    else if (name == "feature_projection/adam_m") { buf = &E.proj_m; row0 = net * E.Fp; }
    else if (name == "feature_projection/adam_v") { buf = &E.proj_v; row0 = net * E.Fp; }
    const size_t rows = var->shape[0], cols = var->shape[1];
    if (rows == 0 || cols == 0) return;
    HIP_CHECK(hipStreamSynchronize(E.stream));
    if (name.rfind("mlp_", 0) == 0) {
        const bool is_up = name.rfind("mlp_up_projection", 0) == 0;
        const bool m = name.size() > 7 && name.compare(name.size() - 7, 7, "/adam_m") == 0;
        const bool v = name.size() > 7 && name.compare(name.size() - 7, 7, "/adam_v") == 0;
        float* dev = is_up ? (m ? E.up_m.p : v ? E.up_v.p : E.up.p) : (m ? E.down_m.p : v ? E.down_v.p : E.down.p);
        dev += net * (is_up ? 2 * (size_t)E.Dp * E.mlp : (size_t)E.mlp * E.Dp);
        // Up: host rows [0, D) and [D, 2 D) are device rows [0, D) and [Dp, Dp + D), pitch M;
        // Down: host [M, D] in device rows of pitch Dp
        const size_t D = E.D, Dp = E.Dp, M = E.mlp;
        for (int half = 0; half < (is_up ? 2 : 1); ++half) {
            float* d = dev + (is_up ? (size_t)half * Dp * M : 0);
            float* h = host + (is_up ? (size_t)half * D * M : 0);
            const size_t dpitch = (is_up ? M : Dp) * 4, hpitch = cols * 4, n = is_up ? D : M;
            if (write) HIP_CHECK(hipMemcpy2D(d, dpitch, h, hpitch, cols * 4, n, hipMemcpyHostToDevice));
            else HIP_CHECK(hipMemcpy2D(h, hpitch, d, dpitch, cols * 4, n, hipMemcpyDeviceToHost));
        }
        return;
    }
    if (write)
        HIP_CHECK(hipMemcpy2D(buf->p + row0 * E.Dp, (size_t)E.Dp * 4, host, cols * 4, cols * 4, rows, hipMemcpyHostToDevice));
    else
        HIP_CHECK(hipMemcpy2D(host, cols * 4, buf->p + row0 * E.Dp, (size_t)E.Dp * 4, cols * 4, rows, hipMemcpyDeviceToHost));
}

// ---- entity rows: "write_entity", "read_entity" (:857-871) --------------------

void upload_row_ids(kge_engine& E, const uint32_t* idx, size_t per_shard, std::vector<uint64_t>& rows) {
    rows.resize((size_t)E.S * per_shard);
    for (int s = 0; s < E.S; ++s)
        for (size_t i = 0; i < per_shard; ++i) {
            const uint32_t v = idx[s * per_shard + i];
            if (v >= (uint32_t)E.n_entity) {
                std::ostringstream msg;
                msg << "entity index " << v << " out of range [0, " << E.n_entity << ")";
                throw std::invalid_argument(msg.str());
            }
            rows[s * per_shard + i] = (E.shared_table ? 0 : (uint64_t)s * E.n_entity) + v;
        }
    HIP_CHECK(hipMemcpyAsync(E.io_rows.p, rows.data(), rows.size() * 8, hipMemcpyHostToDevice, E.stream));
}

void run_write_entity(kge_engine& E, const Items& in, bool raw) {
    const size_t S = E.S, rw = E.rw_batch, W = raw ? 3 * E.D + E.F : E.F;
    const uint32_t* idx = (const uint32_t*)in.array("write_indices", KGE_U32, {S, rw});
    const int kind = raw ? KGE_F32 : E.stream_kind;
    const void* data = in.array(raw ? "write_data" : "write_features", kind, {S, rw, W});
    std::vector<uint64_t> rows;
    upload_row_ids(E, idx, rw, rows);
    std::vector<float> conv;
    const float* src = (const float*)data;
    if (kind == KGE_F16) {
        conv.resize(S * rw * W);
        const uint16_t* h = (const uint16_t*)data;
        for (size_t i = 0; i < conv.size(); ++i) conv[i] = half_to_float(h[i]);
        src = conv.data();
    }
    if (W) HIP_CHECK(hipMemcpyAsync(E.io_data.p, src, S * rw * W * 4, hipMemcpyHostToDevice, E.stream));
    if (raw)
        launch_rows_from_logical(E.L, E.table.p, E.io_rows.p, (int64_t)(S * rw), E.io_data.p, E.stream);
    else  // random-normal embedding with sigma = init_scale / D (:865-866)
        launch_init_rows(E.L, E.table.p, E.io_rows.p, (int64_t)(S * rw), E.io_data.p,
                         E.init_scale / (float)E.D, E.seed, E.stream);
    HIP_CHECK(hipGetLastError());
    HIP_CHECK(hipStreamSynchronize(E.stream));
}

void run_read_entity(kge_engine& E, const Items& in) {
    const size_t S = E.S, rw = E.rw_batch, W = 3 * E.D + E.F;
    const uint32_t* idx = (const uint32_t*)in.array("read_indices", KGE_U32, {S, rw});
    void* out = in.array("read_data", E.stream_kind, {S, rw, W});
    std::vector<uint64_t> rows;
    upload_row_ids(E, idx, rw, rows);
    launch_rows_to_logical(E.L, E.table.p, E.io_rows.p, (int64_t)(S * rw), E.io_data.p, E.stream);
    HIP_CHECK(hipGetLastError());
    if (E.stream_kind == KGE_F32) {
        HIP_CHECK(hipMemcpyAsync(out, E.io_data.p, S * rw * W * 4, hipMemcpyDeviceToHost, E.stream));
        HIP_CHECK(hipStreamSynchronize(E.stream));
    } else {
        std::vector<float> tmp(S * rw * W);
        HIP_CHECK(hipMemcpyAsync(tmp.data(), E.io_data.p, tmp.size() * 4, hipMemcpyDeviceToHost, E.stream));
        HIP_CHECK(hipStreamSynchronize(E.stream));
        uint16_t* h = (uint16_t*)out;
        for (size_t i = 0; i < tmp.size(); ++i) h[i] = float_to_half(tmp[i]);
    }
}

// ---- training ------------------------------------------------------------------

struct BatchPtrs {
    const uint32_t *remote, *a2a, *head, *relation, *tail;
};

BatchPtrs bind_batch(kge_engine& E, const Items& in) {
    const size_t S = E.S, ns = E.n_step;
    BatchPtrs b;
    b.remote = (const uint32_t*)in.array("remote", KGE_U32, {S, ns, (size_t)E.NR});
    b.a2a = (const uint32_t*)in.array("a2a", KGE_U32, {S, ns, S, (size_t)E.A});
    b.head = (const uint32_t*)in.array("head", KGE_U32, {S, ns, (size_t)E.B});
    b.relation = (const uint32_t*)in.array("relation", KGE_U32, {S, ns, (size_t)E.B});
    b.tail = (const uint32_t*)in.array("tail", KGE_U32, {S, ns, (size_t)E.B});
    return b;
}

// Steps [s0, s0 + sn) of the caller's arrays ([S, n_step, ...] each) into the pinned staging
// buffer in the device's step-by-step layout.  Every index a kernel will dereference is checked
// here, on the host, while it passes through.
void stage_steps(kge_engine& E, const BatchPtrs& b, int s0, int sn) {
    const size_t S = E.S, ns = E.n_step;
    struct Part { const char* name; const uint32_t* src; size_t width, offset; uint32_t limit; };
    const Part parts[5] = {
        {"remote", b.remote, (size_t)E.NR, 0, (uint32_t)E.n_entity},
        {"a2a", b.a2a, S * E.A, E.off_a2a, (uint32_t)E.NR},
        {"head", b.head, (size_t)E.B, E.off_head, (uint32_t)E.NR},
        {"relation", b.relation, (size_t)E.B, E.off_relation, (uint32_t)E.n_rel},
        {"tail", b.tail, (size_t)E.B, E.off_tail, (uint32_t)E.T},
    };
    for (int i = s0; i < s0 + sn; ++i) {
        uint32_t* step_block = E.h_idx + (size_t)i * E.idx_words;
        for (const Part& p : parts) {
            // v < limit for every word, without a compare per word: with limit <= 2^31 the top bit
            // of v | (limit - 1 - v) is set exactly when v >= limit
            const uint32_t lm1 = p.limit - 1u;
            uint32_t acc = 0;
            for (size_t s = 0; s < S; ++s) {
                const uint32_t* src = p.src + (s * ns + (size_t)i) * p.width;
                uint32_t* dst = step_block + p.offset + s * p.width;
                for (size_t x = 0; x < p.width; ++x) {
                    const uint32_t v = src[x];
                    dst[x] = v;
                    acc |= v | (lm1 - v);
                }
            }
            uint32_t worst = 0;
            if (acc >> 31)
                for (size_t s = 0; s < S; ++s)
                    for (size_t x = 0; x < p.width; ++x)
                        worst = std::max(worst, p.src[(s * ns + (size_t)i) * p.width + x]);
            if (worst >= p.limit) {
                std::ostringstream msg;
                msg << "'" << p.name << "' holds index " << worst << " out of range [0, " << p.limit << ") (step " << i << ")";
                throw std::invalid_argument(msg.str());
            }
        }
    }
}

// the staged steps' upload
void upload_steps(kge_engine& E, int s0, int sn, hipStream_t st) {
    HIP_CHECK(hipMemcpyAsync(E.d_idx.p + (size_t)s0 * E.idx_words, E.h_idx + (size_t)s0 * E.idx_words,
                             (size_t)sn * E.idx_words * 4, hipMemcpyHostToDevice, st));
}

struct KernelTimer {
    kge_engine& E;
    int id;
    KernelTimer(kge_engine& e, int id_) : E(e), id(id_) {
        if (E.profile_kernels) push();
    }
    ~KernelTimer() {
        if (E.profile_kernels) push();
    }
    void push() {
        hipEvent_t ev;
        (void)hipEventCreate(&ev);
        (void)hipEventRecord(ev, E.stream);
        E.kev.push_back(ev);
        E.kev_id.push_back(id);
    }
};

void collect_kernel_times(kge_engine& E) {
    for (size_t i = 0; i + 1 < E.kev.size(); i += 2) {
        float ms = 0.f;
        (void)hipEventElapsedTime(&ms, E.kev[i], E.kev[i + 1]);
        E.kernel_ms[E.kev_id[i]] += ms;
        E.kernel_calls[E.kev_id[i]] += 1;
    }
    for (auto& e : E.kev) (void)hipEventDestroy(e);
    E.kev.clear();
    E.kev_id.clear();
}

// Index-only work for steps [s0, s0 + sn) of the resident batch: contribution
// keys, the two sorts and the segment / chunk tables.
void run_plan(kge_engine& E, int s0, int sn, hipStream_t st) {
    KernelTimer timer(E, K_PLAN);  // (events on the engine's stream: meaningful when st is that stream)
    const size_t R = E.R, SB = (size_t)E.S * E.B, N = 2 * R, NRI = E.n_rel_items;
    PlanShape ps;
    ps.n_step = E.n_step; ps.S = E.S; ps.B = E.B; ps.A = E.A; ps.NR = E.NR;
    ps.n_entity = E.n_entity; ps.shared_table = E.shared_table; ps.n_relation = E.n_rel;
    ps.rel_copies = E.rel_copies;
    ps.step0 = s0; ps.step_count = sn;
    ps.idx_step_stride = (int64_t)E.idx_words;
    ps.merge_tails = E.merge_tails ? 1 : 0;
    const int ebits = std::max(1, bit_length((uint64_t)E.n_rows - 1)) + kKeyFlagBits;
    const int rbits = std::max(1, bit_length((uint64_t)E.n_rel_rows - 1)) + kKeyFlagBits;
    // both sorts in shared launches, the first pass's histograms from the item kernel
    uint32_t* const e_hist = E.hist.p;
    uint32_t* const r_hist = E.hist.p + radix_sort_hist_words((int)N, E.n_step, std::max(ebits, rbits));
    if (E.merge_tails)
        launch_merge_tails(ps, E.d_idx.p, E.d_idx.p + E.off_a2a, E.tkey.p, E.tmult.p, E.tcol.p, E.tcount.p, st);
    launch_build_items(ps, E.d_idx.p, E.d_idx.p + E.off_a2a, E.d_idx.p + E.off_head, E.d_idx.p + E.off_relation,
                       E.d_idx.p + E.off_tail, E.tkey.p, E.tcol.p, E.ckey.p,
                       E.crel.p, E.clabel.p, E.ek_a.p, E.ev_a.p, E.rk_a.p, E.rv_a.p,
                       sort_passes(std::max(ebits, rbits)).bits[0], e_hist, r_hist, st);
    SortBuffers es = {}, rs = {};
    es.keys_a = E.ek_a.p + s0 * N; es.vals_a = E.ev_a.p + s0 * N; es.keys_b = E.ek_b.p + s0 * N; es.vals_b = E.ev_b.p + s0 * N;
    es.hist = e_hist; es.N = (int)N; es.key_bits = ebits;
    rs.keys_a = E.rk_a.p + s0 * NRI; rs.vals_a = E.rv_a.p + s0 * NRI; rs.keys_b = E.rk_b.p + s0 * NRI; rs.vals_b = E.rv_b.p + s0 * NRI;
    rs.hist = r_hist; rs.N = (int)NRI; rs.key_bits = rbits;
    launch_radix_sort2(&es, &rs, sn, true, st);
    const uint32_t* ek = es.result_in_b ? E.ek_b.p : E.ek_a.p;
    E.e_sorted_vals = es.result_in_b ? E.ev_b.p : E.ev_a.p;
    SegJob ej = {};
    ej.keys = ek + s0 * N; ej.vals = E.e_sorted_vals + s0 * N;
    ej.N = (int)N; ej.n_real = (int)R; ej.chunk = E.chunk; ej.direct_max = E.direct_max;
    SegPlan& ep = ej.plan;
    ep.u_stride = E.e_ustride; ep.c_stride = E.e_cstride;
    ep.uniq_key = E.e_uniq.p + (size_t)s0 * ep.u_stride;
    ep.seg_start = E.e_seg.p + (size_t)s0 * (ep.u_stride + 1);
    ep.chunk_off = E.e_coff.p + (size_t)s0 * (ep.u_stride + 1);
    ep.chunk_pos = E.e_cpos.p + (size_t)s0 * ep.c_stride;
    ep.chunk_len = E.e_clen.p + (size_t)s0 * ep.c_stride;
    ep.counts = E.e_counts.p + 2 * (size_t)s0;
    ep.item_row = E.F ? E.e_item_row.p + s0 * R : nullptr;
    ep.seg_real = E.e_real.p + (size_t)s0 * ep.u_stride;
    ep.hot_rows = E.e_hot.p + (size_t)s0 * ep.c_stride; ep.hot_count = E.e_hot_count.p + 2 * s0;
    ep.chunk_row = E.e_crow.p + (size_t)s0 * ep.c_stride;
    ep.host_counts = E.d_e_counts + 4 * (size_t)s0;

    const uint32_t* rk = rs.result_in_b ? E.rk_b.p : E.rk_a.p;
    E.r_sorted_vals = rs.result_in_b ? E.rv_b.p : E.rv_a.p;
    SegJob rj = {};
    rj.keys = rk + s0 * NRI; rj.vals = E.r_sorted_vals + s0 * NRI;
    rj.N = (int)NRI; rj.n_real = (int)SB * E.rel_copies; rj.chunk = E.chunk; rj.direct_max = E.direct_max;
    SegPlan& rp = rj.plan;
    rp.u_stride = E.r_ustride; rp.c_stride = E.r_cstride;
    rp.uniq_key = E.r_uniq.p + (size_t)s0 * rp.u_stride;
    rp.seg_start = E.r_seg.p + (size_t)s0 * (rp.u_stride + 1);
    rp.chunk_off = E.r_coff.p + (size_t)s0 * (rp.u_stride + 1);
    rp.chunk_pos = E.r_cpos.p + (size_t)s0 * rp.c_stride;
    rp.chunk_len = E.r_clen.p + (size_t)s0 * rp.c_stride;
    rp.counts = E.r_counts.p + 2 * (size_t)s0;
    rp.item_row = nullptr;
    rp.seg_real = E.r_real.p + (size_t)s0 * rp.u_stride;
    rp.hot_rows = E.r_hot.p + (size_t)s0 * rp.c_stride; rp.hot_count = E.r_hot_count.p + 2 * s0;
    rp.chunk_row = E.r_crow.p + (size_t)s0 * rp.c_stride;
    rp.host_counts = E.d_r_counts + 4 * (size_t)s0;
    launch_find_segments2(ej, &rj, sn, E.seg_scratch.p, st);  // both plans' segments in one launch
    HIP_CHECK(hipGetLastError());
}

// how the gather combines a head row with its relation row (launch_gather_operands)
static int rel_mode_of(const kge_engine& E) {
    if (E.score_fn == SCORE_TRANSH) return 0;  // launch_transh_predict turns the copied head rows into p
    return E.score_fn == SCORE_DISTMULT ? 2 : E.score_fn == SCORE_COMPLEX ? 3 : E.score_fn == SCORE_ROTATE ? 4 : 1;
}

void run_step(kge_engine& E, int i) {
    const hipStream_t st = E.stream;
    const size_t R = E.R, SB = (size_t)E.S * E.B;
    ScoreShape sh;
    sh.S = E.S; sh.B = E.B; sh.T = E.T; sh.Dp = E.Dp;
    sh.score_fn = E.score_fn; sh.dist_fn = E.dist_fn; sh.loss_fn = E.loss_fn;
    sh.gamma = E.gamma; sh.loss_scale = E.loss_scale;
    sh.softmax_correction = 0.f;
    if (E.loss_fn == LOSS_SOFTMAX && E.softmax_cw != 0.f) {
        // src/poplar_kge.cpp:644: float correction = log(nEntity*nShard - 1) - log(nShard*a2aSize - 1)
        const float corr = (float)(std::log((double)((uint32_t)E.n_entity * (uint32_t)E.S - 1u)) -
                                   std::log((double)((uint32_t)E.S * (uint32_t)E.A - 1u)));
        sh.softmax_correction = E.softmax_cw * corr;
    }
    sh.negative_adversarial_scale = E.neg_adv;
    sh.use_mfma = E.use_mfma;
    sh.operands_dense = 0;
    sh.tcount = E.merge_tails ? E.tcount.p + (size_t)i * E.S : nullptr;
    sh.tmult = E.merge_tails ? E.tmult.p + (size_t)i * E.S * E.T : nullptr;
    sh.tpad = E.tpad;
    const bool fused = E.loss_fn == LOSS_LOGSIGMOID && E.neg_adv <= 0.f && !E.score_bf16;

    const uint32_t* ckey = E.ckey.p + i * R;
    const uint32_t* crel = E.crel.p + i * SB;
    const uint32_t* clabel = E.clabel.p + i * SB;
    const uint32_t* e_counts = E.e_counts.p + 2 * (size_t)i;
    const uint32_t* e_uniq = E.e_uniq.p + (size_t)i * E.e_ustride;
    const uint32_t* r_counts = E.r_counts.p + 2 * (size_t)i;

    RowSource table_rows;  // entity embeddings straight from the table
    table_rows.base = E.table.p; table_rows.pitch = E.L.pitch; table_rows.etype = E.L.emb_etype;
    table_rows.index = ckey; table_rows.count = E.Dp; table_rows.vec = 1;
    RowSource ent = table_rows;

    // Feature path.  One feature network, or a head and a tail one (index 0 / 1 of fa, ma and
    // of every per-network buffer).  A distinct row has one hidden row, or two (its use as a head,
    // its use as a tail) when the networks are separate or with dropout.
    FeatureArgs fa[2] = {};
    MlpArgs ma[2] = {};
    DropoutArgs da = {};
    const int nets = E.nets;
    const bool drop = E.dropout > 0, roles = E.F && (drop || nets == 2);
    const size_t rows_n = R * (size_t)E.Dp;  // elements of one per-row buffer
    if (E.F) {
        KernelTimer t(E, K_HIDDEN);
        for (int net = 0; net < nets; ++net) {
            FeatureArgs& f = fa[net];
            f.uniq_key = e_uniq; f.counts = e_counts; f.max_rows = (int)R;
            f.emb_base = E.table.p; f.feat_base = E.table.p + E.L.off_f; f.pitch = E.L.pitch;
            f.emb_etype = E.L.emb_etype; f.feat_etype = E.L.feat_etype;
            f.Dp = E.Dp; f.Fp = E.Fp; f.proj = E.proj.p + (size_t)net * E.Fp * E.Dp;
            f.featd = E.featd.p; f.gproj_part = E.gproj_part.p; f.use_mfma = E.use_mfma;
            f.round_bf16 = E.score_bf16 ? 1 : 0; f.projR = E.projR.p;
            f.feat16 = E.feat16.p;
            FeatureArgs fp = f;  // the feature part alone, without the embedding
            fp.emb_base = nullptr;
            float* hid = E.hidden.p + net * rows_n;          // value + feature part
            float* part = drop ? E.fh.p + net * rows_n : hid;  // what this network's kernels write
            if (E.mlp) {  // feature . W alone, then the MLP on [embedding | feature . W]
                MlpArgs& m = ma[net];
                float* fproj = E.mlp_fproj.p + net * rows_n;
                launch_hidden_fwd(fp, fproj, st);
                m.uniq_key = e_uniq; m.counts = e_counts; m.max_rows = (int)R;
                m.emb_base = E.table.p; m.pitch = E.L.pitch; m.emb_etype = E.L.emb_etype;
                m.Dp = E.Dp; m.M = E.mlp;
                m.up = E.up.p + (size_t)net * 2 * E.Dp * E.mlp; m.down = E.down.p + (size_t)net * E.mlp * E.Dp;
                m.concat = E.mlp_concat.p + 2 * net * rows_n; m.pre = E.mlp_pre.p + (size_t)net * R * E.mlp;
                m.add_value = drop ? 0 : 1;
                launch_mlp_fwd(m, fproj, part, st);
            } else {
                launch_hidden_fwd(drop ? fp : f, part, st);
            }
        }
        ent.base = (const char*)E.hidden.p; ent.pitch = (int64_t)E.Dp * 4; ent.etype = ET_F32;
        ent.index = E.e_item_row.p + i * R;
        if (roles) {
            da.uniq_key = e_uniq; da.counts = e_counts; da.max_rows = (int)R;
            da.emb_base = E.table.p; da.pitch = E.L.pitch; da.emb_etype = E.L.emb_etype; da.Dp = E.Dp;
            da.seed = E.seed; da.step = (uint32_t)(E.step_of_first + i);
            da.threshold = (uint32_t)((double)E.dropout * 4294967296.0);
            da.scale = drop ? 1.f / (1.f - E.dropout) : 1.f;
            da.enabled = drop ? 1 : 0;
            // with dropout (src/poplar_kge.cpp:459-461, once per entityHidden call) the two hidden
            // rows are formed here; every contribution reads the one of its role
            if (drop) launch_dropout_hidden(da, E.fh.p, E.fh.p + (nets - 1) * rows_n, E.hidden.p, st);
            launch_role_index(E.e_item_row.p + i * R, (int)SB, (int)R, E.role_idx.p, st);
            ent.index = E.role_idx.p;
        }
    }

    // dense operands: every contribution's row, float32, relation applied to the heads
    { KernelTimer t(E, K_GATHER);
      TailCols tc = {sh.tcount, E.T, E.tpad};
      launch_gather_operands(ent, E.rel.p, crel, rel_mode_of(E), E.D / 2, (int)SB, (int)R, E.Dp,
                             E.opnd.p, E.score_bf16 ? E.opnd16.p : nullptr, st, &tc); }
    RowSource dense;
    dense.base = (const char*)E.opnd.p; dense.pitch = (int64_t)E.Dp * 4; dense.etype = ET_F32;
    dense.index = nullptr; dense.count = E.Dp; dense.vec = 1;
    sh.operands_dense = 1;
    const bool transh = E.score_fn == SCORE_TRANSH;
    if (transh) {
        // second operand matrix [unit normals | tails]; the heads of the first become the
        // predicted tails (transHPredict, src/poplar_kge.cpp:539-549)
        KernelTimer t(E, K_GATHER);
        HIP_CHECK(hipMemcpyAsync(E.opnd_n.p, E.opnd.p, R * E.Dp * 4, hipMemcpyDeviceToDevice, st));
        launch_transh_predict(E.rel.p, crel, E.n_rel, (int)SB, E.Dp, E.opnd.p, E.opnd_n.p, st);
    }

    float* loss_part = E.loss_part.p + (size_t)i * E.S * E.n_part;
    // bfloat16 dot-product scoring on the matrix cores: three batched products
    //   scores = q . tails^T,   d q = c . tails,   d tails = c^T . q
    const int Bn = E.B, Tn = E.T, Dp = E.Dp;
    const bool bf16_fast = E.score_bf16 && E.use_mfma && gemm_nt_bf16_ok(Bn, Tn, Dp) &&
                           gemm_nt_bf16_ok(Bn, Dp, Tn) && gemm_nt_bf16_ok(Tn, Dp, Bn);
    if (bf16_fast) {
        const size_t head_n = SB * (size_t)Dp;
        GemmNT g = {};
        g.batches = E.S;
        // merged tails: block d's live tail columns end at its distinct count (whole tiles)
        const uint32_t* const tc = sh.tcount;
        g.limit_stride = 1;
        { KernelTimer t(E, K_FWD);
          g.A = E.opnd16.p; g.lda = Dp; g.a_batch = (int64_t)Bn * Dp;
          g.Bt = E.opnd16.p + head_n; g.ldb = Dp; g.b_batch = (int64_t)Tn * Dp;
          g.C = E.coef.p; g.ldc = Tn; g.c_batch = (int64_t)Bn * Tn;
          g.M = Bn; g.N = Tn; g.K = Dp;
          g.n_limit = tc;
          launch_gemm_nt_bf16(g, st);
          g.n_limit = nullptr; }
        // only the bfloat16 coefficients are read from here on
        { KernelTimer t(E, K_LOSS); launch_loss_rows(sh, clabel, E.coef.p, nullptr, loss_part, E.coef16.p, st, false); }
        // d q and d tails contract over the rows of their second operand (and d tails over the
        // rows of the coefficients too): the product kernel takes such operands as they lie
        { KernelTimer t(E, K_BWD);
          // d q [B, Dp] = c [B, T] . tails [T, Dp]
          g.A = E.coef16.p; g.lda = Tn; g.a_batch = (int64_t)Bn * Tn;
          g.Bt = E.opnd16.p + head_n; g.ldb = Dp; g.b_batch = (int64_t)Tn * Dp; g.b_kmajor = 1;
          g.C = E.grad.p; g.ldc = Dp; g.c_batch = (int64_t)Bn * Dp;
          g.M = Bn; g.N = Dp; g.K = Tn; g.part = E.gemm_part.p;
          g.k_limit = tc;
          launch_gemm_nt_bf16(g, st);
          g.k_limit = nullptr;
          // d tails [T, Dp] = c^T [T, B] . q [B, Dp]
          g.A = E.coef16.p; g.lda = Tn; g.a_batch = (int64_t)Bn * Tn; g.a_kmajor = 1;
          g.Bt = E.opnd16.p; g.ldb = Dp; g.b_batch = (int64_t)Bn * Dp;
          g.C = E.grad.p + head_n; g.ldc = Dp; g.c_batch = (int64_t)Tn * Dp;
          g.M = Tn; g.N = Dp; g.K = Bn;
          g.m_limit = tc;
          launch_gemm_nt_bf16(g, st); }
    } else if (transh) {
        // transHScore (:551-565): c = n . tail and its backward are dot-product scoring on
        // [normals | tails]; the L1 part has kernels of its own
        RowSource dense_n = dense;
        dense_n.base = (const char*)E.opnd_n.p;
        ScoreShape dot = sh;
        dot.score_fn = SCORE_DISTMULT; dot.dist_fn = DIST_DOT;
        { KernelTimer t(E, K_FWD);
          launch_score_fwd(dot, dense_n, E.rel.p, crel, clabel, E.cmat.p, nullptr, nullptr, nullptr, false, st);
          TranshFwd tf;
          tf.sh = sh; tf.pt = E.opnd.p; tf.nt = E.opnd_n.p; tf.cmat = E.cmat.p; tf.clabel = clabel;
          tf.coef = E.coef.p; tf.dcm = E.dcm.p; tf.loss_part = loss_part;
          launch_transh_fwd(tf, fused, st); }
        if (!fused) {
            KernelTimer t(E, K_LOSS);
            launch_loss_rows(sh, clabel, E.coef.p, nullptr, loss_part, nullptr, st);
            launch_mul_rows(E.dcm.p, E.coef.p, (int64_t)SB * E.T, st);
        }
        { KernelTimer t(E, K_BWD);
          launch_score_bwd(dot, dense_n, E.rel.p, crel, E.dcm.p, nullptr, E.transh_mm.p, st);
          TranshBwd tb;
          tb.pt = E.opnd.p; tb.nt = E.opnd_n.p; tb.coef = E.coef.p; tb.cmat = E.cmat.p;
          tb.mm = E.transh_mm.p; tb.grad = E.grad.p; tb.S = E.S; tb.B = E.B; tb.T = E.T; tb.Dp = E.Dp;
          launch_transh_bwd(tb, st);
          launch_transh_back(ent, E.rel.p, crel, E.n_rel, (int)SB, E.Dp, E.grad.p, E.transh_mm.p, E.relgrad.p, st); }
    } else {
        { KernelTimer t(E, K_FWD);
          launch_score_fwd(sh, dense, E.rel.p, crel, clabel, E.coef.p, E.dist.p, E.nearflag.p, loss_part, fused, st); }
        if (!fused) { KernelTimer t(E, K_LOSS); launch_loss_rows(sh, clabel, E.coef.p, E.dist.p, loss_part, nullptr, st); }
        { KernelTimer t(E, K_BWD); launch_score_bwd(sh, dense, E.rel.p, crel, E.coef.p, E.nearflag.p, E.grad.p, st); }
    }

    if (E.reg_on) {
        RegArgs ra = {};
        ra.uniq_key = e_uniq; ra.counts = e_counts; ra.max_rows = (int)R;
        ra.seg_start = E.e_seg.p + (size_t)i * (E.e_ustride + 1);
        ra.seg_real = E.e_real.p + (size_t)i * E.e_ustride;
        ra.emb_base = E.table.p; ra.pitch = E.L.pitch; ra.emb_etype = E.L.emb_etype;
        ra.hidden = E.F ? E.hidden.p : nullptr;
        ra.D = E.D; ra.Dp = E.Dp;
        for (int q = 0; q < 3; ++q) { ra.power[q] = E.reg_p[q]; ra.weight[q] = E.reg_w[q]; }
        ra.loss_scale = E.loss_scale;
        ra.add_val = E.reg_val.p; ra.add_fh = E.reg_fh.p; ra.loss_row = E.reg_loss_row.p;
        ra.uses = 2.f; ra.accumulate = 0;
        if (roles) {  // the two entityHidden calls see different rows: one launch for each
            ra.uses = 1.f;
            launch_reg_rows(ra, st);
            ra.hidden = E.hidden.p + rows_n; ra.add_fh = E.reg_fh.p + rows_n; ra.accumulate = 1;
        }
        launch_reg_rows(ra, st);
        launch_reg_loss(e_uniq, e_counts, E.reg_loss_row.p, (uint32_t)E.n_entity, E.S,
                        E.reg_loss_part.p + (size_t)i * E.S, st);
    }

    if (E.counts_pending) {  // the plan's counts size the launches from here on
        HIP_CHECK(hipEventSynchronize(E.counts_wait));
        E.counts_pending = false;
    }
    const float* alpha = E.d_alpha.p + (size_t)i * 9 * E.S;
    AdamArgs aa = {};
    aa.Dp = E.Dp;
    aa.beta_m = E.beta_m; aa.beta_v = E.beta_v;
    aa.one_minus_beta_m = 1.f - E.beta_m; aa.one_minus_beta_v = 1.f - E.beta_v;
    aa.epsilon = E.epsilon; aa.weight_decay = E.weight_decay;

    // both reductions read pre-update rows (DistMult and ComplEx multiply by them), so they
    // come before both updates
    ContribSrc rsrc = {};
    rsrc.sorted_item = E.r_sorted_vals + (size_t)i * E.n_rel_items;
    rsrc.grad = transh ? E.relgrad.p : E.grad.p;  // TransH: rows [0, SB) embedding, [SB, 2 SB) normal contributions
    rsrc.transform = E.score_fn == SCORE_DISTMULT ? 2 : E.score_fn == SCORE_COMPLEX ? 4 : E.score_fn == SCORE_ROTATE ? 6 : 0;
    rsrc.n_head = (int)SB; rsrc.half = E.D / 2;
    rsrc.rel = E.rel.p; rsrc.crel = crel; rsrc.ent = ent;
    ContribSrc esrc = rsrc;
    esrc.sorted_item = E.e_sorted_vals + (size_t)i * 2 * R;
    esrc.grad = E.grad.p;
    esrc.transform = E.score_fn == SCORE_DISTMULT ? 1 : E.score_fn == SCORE_COMPLEX ? 3 : E.score_fn == SCORE_ROTATE ? 5 : 0;

    ReduceArgs rr = {};
    rr.src = rsrc;
    rr.chunk_pos = E.r_cpos.p + (size_t)i * E.r_cstride;
    rr.chunk_len = E.r_clen.p + (size_t)i * E.r_cstride;
    rr.counts = r_counts; rr.max_chunks = E.r_cstride; rr.chunk = E.chunk;
    if (E.counts_known) rr.max_chunks = (int)E.h_r_counts[4 * (size_t)i + 1];
    rr.partial = E.rel_partial.p; rr.Dp = E.Dp;

    ReduceArgs re = {};
    re.src = esrc;
    re.chunk_pos = E.e_cpos.p + (size_t)i * E.e_cstride;
    re.chunk_len = E.e_clen.p + (size_t)i * E.e_cstride;
    re.counts = e_counts; re.max_chunks = E.e_cstride; re.chunk = E.chunk;
    if (E.counts_known) re.max_chunks = (int)E.h_e_counts[4 * (size_t)i + 1];
    re.partial = E.partial.p; re.Dp = E.Dp;
    // Contributions used as stored, nothing between the sums and the updates, and no row with
    // more contributions than a handful of workgroups sum in the time the other rows take (known
    // from the plan's read-back): the rows with chunks are summed and updated by workgroups of
    // their own inside the update's launch, and the first-level reduction (a launch whose time
    // is all latency) is not needed.  A row of 5 600 contributions (the 22.8M-row workload's
    // hottest) takes its eight workgroups longer than the whole update takes otherwise; one of
    // 2 200 (the 1M-row workload's) fits under it.
    const bool hot_in_update = !contributions_read_tables(E) && !E.mlp && !roles && E.counts_known &&
                               std::max(E.h_e_counts[4 * (size_t)i + 3], E.h_r_counts[4 * (size_t)i + 3]) <= kHotInUpdateMax;
    if (!hot_in_update) { KernelTimer t(E, K_REDUCE_ENT); launch_reduce_chunks2(re, rr, st); }

    // With DistMult / ComplEx the relation rows' direct contributions read entity rows and
    // the entity rows' read relation rows, so neither table may be updated before
    // the other's gradient is complete: materialise the relation gradient first.
    // (TransE contributions do not depend on either table.)
    AdamArgs ar = aa;
    ar.src = rsrc;
    ar.uniq_key = E.r_uniq.p + (size_t)i * E.r_ustride;
    ar.seg_start = E.r_seg.p + (size_t)i * (E.r_ustride + 1);
    ar.seg_real = E.r_real.p + (size_t)i * E.r_ustride;
    ar.chunk_off = E.r_coff.p + (size_t)i * (E.r_ustride + 1);
    ar.counts = r_counts; ar.max_rows = E.n_rel_rows;
    ar.partial = E.rel_partial.p;
    ar.p_base = (char*)E.rel.p; ar.m_base = (char*)E.rel_m.p; ar.v_base = (char*)E.rel_v.p;
    ar.pitch = (int64_t)E.Dp * 4; ar.p_etype = ET_F32; ar.m_etype = ET_F32; ar.v_is_sqrt = 0;
    ar.alpha = alpha + E.S;
    // the normal rows (keys >= n_rel) take the step sizes after the relation embedding's
    ar.rows_per_alpha = E.shared_table ? (transh ? (uint32_t)E.n_rel : 0u) : (uint32_t)(E.n_rel / E.S);

    AdamArgs ae = aa;
    ae.src = esrc;
    ae.uniq_key = e_uniq;
    ae.seg_start = E.e_seg.p + (size_t)i * (E.e_ustride + 1);
    ae.seg_real = E.e_real.p + (size_t)i * E.e_ustride;
    ae.chunk_off = E.e_coff.p + (size_t)i * (E.e_ustride + 1);
    ae.counts = e_counts; ae.max_rows = E.counts_known ? (int)E.h_e_counts[4 * (size_t)i] : (int)R;
    ae.partial = E.partial.p;
    // (with dropout the feature part's gradient is formed per role by launch_role_sums)
    ae.grad_out = (E.F && !roles) ? E.gsum.p : nullptr;
    if (E.reg_on) { ae.grad_add = E.reg_val.p; ae.grad_out_add = E.reg_fh.p; }
    ae.p_base = E.table.p; ae.m_base = E.table.p + E.L.off_m; ae.v_base = E.table.p + E.L.off_s;
    ae.pitch = E.L.pitch; ae.p_etype = E.L.emb_etype; ae.m_etype = E.L.mom_etype; ae.v_is_sqrt = 1;
    ae.alpha = alpha;
    ae.rows_per_alpha = E.shared_table ? 0u : (uint32_t)E.n_entity;

    if (E.keep_gradients) { ae.grad_out = E.gkeep_e.p; ar.grad_out = E.gkeep_r.p; E.last_step = i; }

    // The feature MLP's input holds the embedding, so part of the embedding's gradient comes
    // back through the MLP: the rows' summed gradient first (a pass without update), the MLP's
    // backward per row, then the update with what that adds.
    auto entity_update = [&]() {
        KernelTimer t(E, K_ADAM_ENT);
        if (roles)  // the feature part's gradient per use: one array (added up) or one per network
            launch_role_sums(da, esrc, ae.seg_start, ae.seg_real, E.fh.p, E.fh.p + (nets - 1) * rows_n,
                             E.reg_on ? E.reg_fh.p : nullptr, E.reg_on ? E.reg_fh.p + rows_n : nullptr, E.gsum.p,
                             nets == 2 ? E.gsum.p + rows_n : nullptr, st);
        if (!E.mlp) { launch_adam_rows(ae, st); return; }
        if (!roles) {
            AdamArgs sum = ae;
            sum.no_update = 1;
            launch_adam_rows(sum, st);
        }
        for (int net = 0; net < nets; ++net)  // what reaches the embedding adds up over the networks
            launch_mlp_bwd_rows(ma[net], E.gsum.p + net * rows_n,
                                net ? E.mlp_gval.p : (E.reg_on ? E.reg_val.p : nullptr),
                                E.mlp_gpre.p + (size_t)net * R * E.mlp, E.mlp_gval.p, E.mlp_gfp.p + net * rows_n, st);
        AdamArgs upd = ae;
        upd.grad_out = nullptr; upd.grad_out_add = nullptr; upd.grad_add = E.mlp_gval.p;
        launch_adam_rows(upd, st);
    };
    if (contributions_read_tables(E)) {
        // entity update first (reads pre-update relation rows), writing its summed
        // gradient is not needed; then the relation update reads POST-update entity
        // rows unless its gradient was materialised: do that with a zero-step pass
        ar.grad_out = E.rel_gsum.p;
        ar.no_update = 1;
        if (E.F && !E.mlp && !roles) {
            // with entity features the relation rows' contributions read the hidden rows formed
            // at the start of the step, not the table: their sum can share the entity update's launch
            KernelTimer t(E, K_ADAM_ENT);
            launch_adam_rows2(ar, ae, st);
        } else {
            { KernelTimer t(E, K_ADAM_REL); launch_adam_rows(ar, st); }
            entity_update();
        }
        ar.grad_out = nullptr; ar.no_update = 0;
        ar.grad_direct = E.rel_gsum.p;
        { KernelTimer t(E, K_ADAM_REL); launch_adam_rows(ar, st); }
    } else if (E.mlp || roles) {
        entity_update();
        KernelTimer t(E, K_ADAM_REL);
        launch_adam_rows(ar, st);
    } else if (hot_in_update) {
        KernelTimer t(E, K_ADAM_ENT);
        HotRows he, hr;
        he.hot_rows = E.e_hot.p + (size_t)i * E.e_cstride; he.hot_count = E.e_hot_count.p + 2 * i;
        he.max_hot = (int)E.h_e_counts[4 * (size_t)i + 2];
        hr.hot_rows = E.r_hot.p + (size_t)i * E.r_cstride; hr.hot_count = E.r_hot_count.p + 2 * i;
        hr.max_hot = (int)E.h_r_counts[4 * (size_t)i + 2];
        he.chunk_row = E.e_crow.p + (size_t)i * E.e_cstride; he.n_chunks = (int)E.h_e_counts[4 * (size_t)i + 1];
        hr.chunk_row = E.r_crow.p + (size_t)i * E.r_cstride; hr.n_chunks = (int)E.h_r_counts[4 * (size_t)i + 1];
        launch_adam_rows_hot2(ar, hr, ae, he, st);
    } else {
        // the relation rows first: they are few and slow (a dozen contributions each, two rounds
        // of loads), and at the end of the grid they ran on alone after the entity rows were done
        KernelTimer t(E, K_ADAM_ENT);
        launch_adam_rows2(ar, ae, st);
    }

    // dense Adam on rows [0, rows) of a parameter of row pitch `width`; shard s owns rows
    // [s*rows/S, (s+1)*rows/S) and its step size (group `group` of this step's step sizes)
    auto dense_adam = [&](float* p, float* m, float* v, const float* g, int rows, int last_row, int64_t width,
                          int group) {
        const int n_slices = E.shared_table ? 1 : E.S;
        for (int s = 0; s < n_slices; ++s) {
            const int r0 = E.shared_table ? 0 : s * (rows / E.S);
            const int r1 = (E.shared_table || s == E.S - 1) ? last_row : (s + 1) * (rows / E.S);
            if (r1 <= r0) continue;
            const size_t o = (size_t)r0 * width;
            launch_adam_flat(p + o, m + o, v + o, g + o, (int64_t)(r1 - r0) * width,
                             E.h_alpha[((size_t)i * 9 + group) * E.S + s], E.beta_m, E.beta_v, E.epsilon,
                             E.weight_decay, 0, st);
        }
    };
    for (int net = 0; net < nets && E.F; ++net) {
        const float* g_rows = E.gsum.p + net * rows_n;  // d loss / d (feature part) per distinct row
        if (E.mlp) {
            const size_t up_o = (size_t)net * 2 * E.Dp * E.mlp, down_o = (size_t)net * E.mlp * E.Dp;
            { KernelTimer t(E, K_PROJ_GRAD);
              // d Down = relu(pre)^T . g, d Up = concat^T . gpre, summed over the distinct rows in order
              launch_rows_atb(ma[net].pre, E.mlp, E.mlp, true, g_rows, E.Dp, E.Dp, e_counts, E.g_down.p + down_o, st);
              launch_rows_atb(ma[net].concat, 2 * E.Dp, 2 * E.Dp, false, E.mlp_gpre.p + (size_t)net * R * E.mlp,
                              E.mlp, E.mlp, e_counts, E.g_up.p + up_o, st); }
            KernelTimer t(E, K_ADAM_PROJ);
            // Up's host rows [0, D) and [D, 2 D) are device rows [0, D) and [Dp, Dp + D): a shard's
            // slice of host rows is updated half by half
            const int n_slices = E.shared_table ? 1 : E.S, rows = 2 * E.D;
            for (int s = 0; s < n_slices; ++s) {
                const int r0 = E.shared_table ? 0 : s * (rows / E.S);
                const int r1 = (E.shared_table || s == E.S - 1) ? rows : (s + 1) * (rows / E.S);
                for (int half = 0; half < 2; ++half) {
                    const int lo = std::max(r0, half * E.D), hi = std::min(r1, (half + 1) * E.D);
                    if (hi <= lo) continue;
                    const size_t o = up_o + (size_t)(lo + half * (E.Dp - E.D)) * E.mlp;
                    launch_adam_flat(E.up.p + o, E.up_m.p + o, E.up_v.p + o, E.g_up.p + o, (int64_t)(hi - lo) * E.mlp,
                                     E.h_alpha[((size_t)i * 9 + 4 + 3 * net) * E.S + s], E.beta_m, E.beta_v,
                                     E.epsilon, E.weight_decay, 0, st);
                }
            }
            dense_adam(E.down.p + down_o, E.down_m.p + down_o, E.down_v.p + down_o, E.g_down.p + down_o, E.mlp, E.mlp,
                       E.Dp, 5 + 3 * net);
            g_rows = E.mlp_gfp.p + net * rows_n;  // the projected features' gradient
        }
        const size_t proj_o = (size_t)net * E.Fp * E.Dp;
        { KernelTimer t(E, K_PROJ_GRAD); launch_proj_grad(fa[net], g_rows, E.gproj.p + proj_o, st); }
        KernelTimer t(E, K_ADAM_PROJ);
        dense_adam(E.proj.p + proj_o, E.proj_m.p + proj_o, E.proj_v.p + proj_o, E.gproj.p + proj_o, E.F, E.Fp, E.Dp,
                   3 + 3 * net);
    }
    HIP_CHECK(hipGetLastError());
}

// Engine.train_step_loop's device half (Model::trainStepLoop, :709-741)
void run_train_step_loop(kge_engine& E, const Items& in) {
    const size_t S = E.S;
    const float* lr = (const float*)in.array("learning_rate", KGE_F32, {S});
    float* loss = (float*)in.array("loss", KGE_F32, {S});
    const bool staged = in.find("staged") && in.boolean("staged");
    // additive: run only steps [step_begin, step_begin + step_count) of a staged batch
    int s0 = 0, sn = E.n_step;
    if (in.find("step_begin") || in.find("step_count")) {
        if (!staged) throw std::invalid_argument("'step_begin' / 'step_count' need staged=true");
        s0 = (int)in.uint("step_begin");
        sn = (int)in.uint("step_count");
        if (sn < 1 || s0 + sn > E.n_step) throw std::invalid_argument("step range outside the staged batch");
    }
    const hipStream_t st = E.stream;
    // additive: per-kernel event timing for this call only
    const bool profile_saved = E.profile_kernels;
    if (in.find("profile_kernels")) E.profile_kernels = in.boolean("profile_kernels");
    struct Restore { bool& ref; bool v; ~Restore() { ref = v; } } restore{E.profile_kernels, profile_saved};
    HIP_CHECK(hipEventRecord(E.ev[0], st));
    if (staged && !E.staged) throw std::invalid_argument("train_step_loop with staged=true needs a preceding stage_batch");
    BatchPtrs host = {};
    if (!staged) host = bind_batch(E, in);
    // step sizes of every step of this call (adamStepSizeAutoIncrement, frnn.cpp:42-59)
    E.h_alpha.resize((size_t)E.n_step * 9 * S);
    for (int i = s0; i < s0 + sn; ++i) {
        const double t = (double)(E.step + (uint32_t)(i - s0) + 1u);
        const double factor = std::sqrt(1.0 - std::pow((double)E.beta_v, t)) / (1.0 - std::pow((double)E.beta_m, t));
        for (size_t s = 0; s < S; ++s) {
            const float a = (float)(factor * (double)lr[s]);
            E.h_alpha[((size_t)i * 9 + 0) * S + s] = a * E.lr_mod_entity;
            E.h_alpha[((size_t)i * 9 + 1) * S + s] = a * E.lr_mod_rel;
            E.h_alpha[((size_t)i * 9 + 2) * S + s] = a * E.lr_mod_normal;
            for (int net = 0; net < 2; ++net) {
                E.h_alpha[((size_t)i * 9 + 3 + 3 * net) * S + s] = a * E.lr_mod_proj[net];
                E.h_alpha[((size_t)i * 9 + 4 + 3 * net) * S + s] = a * E.lr_mod_up[net];
                E.h_alpha[((size_t)i * 9 + 5 + 3 * net) * S + s] = a * E.lr_mod_down[net];
            }
        }
        // a shared table has one step size per parameter: the relation update finds the
        // normal rows' at index 1 of its array
        if (E.shared_table && E.score_fn == SCORE_TRANSH)
            E.h_alpha[((size_t)i * 9 + 1) * S + 1] = (float)(factor * (double)lr[0]) * E.lr_mod_normal;
    }
    std::memcpy(E.h_alpha_pin, E.h_alpha.data(), E.h_alpha.size() * 4);
    HIP_CHECK(hipMemcpyAsync(E.d_alpha.p, E.h_alpha_pin, E.h_alpha.size() * 4, hipMemcpyHostToDevice, st));
    HIP_CHECK(hipEventRecord(E.ev[1], st));
    E.step_of_first = (int)E.step - s0;  // step i of the batch is optimiser step E.step + (i - s0)
    // the per-step counts (distinct rows, chunks, rows with chunks, biggest row) size the launches of
    // calls long enough to pay for the wait; the segment kernel writes them into pinned host memory
    E.counts_known = sn >= E.plan_readback_steps;
    E.counts_pending = false;
    if (staged) {
        run_plan(E, s0, sn, st);
        if (E.counts_known) {
            // the host waits for that kernel when the first launch sized by the counts is due, with
            // the first step's scoring launches already queued behind it
            HIP_CHECK(hipEventRecord(E.counts_ready, st));
            E.counts_wait = E.counts_ready;
            E.counts_pending = true;
        }
        HIP_CHECK(hipEventRecord(E.ev[2], st));
        for (int i = s0; i < s0 + sn; ++i) run_step(E, i);
    } else {
        // Host arrays (EngineImpl::runProgram binds them on every run, src/poplar_kge.cpp:967-975):
        // chunks of 2, 4, 8, ... steps.  A helper thread checks and re-orders chunk k + 1 (host
        // memory only) while this thread launches chunk k's kernels; chunk k + 1's upload and
        // plan then run beside chunk k's kernels on streams of their own.  Only the first chunk's
        // preparation is exposed.
        std::vector<std::pair<int, int>> chunks;
        for (int c0 = s0, cn = 2; c0 < s0 + sn; c0 += cn, cn *= 2) {
            cn = std::min(cn, s0 + sn - c0);
            chunks.emplace_back(c0, cn);
        }
        while (E.chunk_copied.size() < chunks.size()) {
            hipEvent_t a = nullptr, b = nullptr;
            HIP_CHECK(hipEventCreateWithFlags(&a, hipEventDisableTiming));
            E.chunk_copied.push_back(a);
            HIP_CHECK(hipEventCreateWithFlags(&b, hipEventDisableTiming));
            E.chunk_planned.push_back(b);
        }
        // the helper: chunks 1 .. n - 1 in order; `ready` counts the chunks staged so far
        std::mutex mu;
        std::condition_variable cv;
        size_t ready = 1;
        std::exception_ptr failed;
        std::thread helper;
        if (chunks.size() > 1)
            helper = std::thread([&]() {
                for (size_t k = 1; k < chunks.size(); ++k) {
                    try {
                        stage_steps(E, host, chunks[k].first, chunks[k].second);
                    } catch (...) {
                        std::lock_guard<std::mutex> lock(mu);
                        failed = std::current_exception();
                        cv.notify_all();
                        return;
                    }
                    std::lock_guard<std::mutex> lock(mu);
                    ready = k + 1;
                    cv.notify_all();
                }
            });
        int done = 0;  // steps handed to the device
        const bool readback = E.counts_known;
        auto enqueue = [&](size_t k) {  // chunk k is staged: its upload and its plan
            if (k == 0) {
                // nothing to run beside: straight onto the engine's stream, and no wait for the
                // plan's counts (the first chunk's launches are sized for the worst case), so
                // that this thread goes on to the next chunk at once
                upload_steps(E, chunks[0].first, chunks[0].second, st);
                run_plan(E, chunks[0].first, chunks[0].second, st);
                HIP_CHECK(hipEventRecord(E.chunk_planned[0], st));
                return;
            }
            upload_steps(E, chunks[k].first, chunks[k].second, E.copy_stream);
            HIP_CHECK(hipEventRecord(E.chunk_copied[k], E.copy_stream));
            HIP_CHECK(hipStreamWaitEvent(E.plan_stream, E.chunk_copied[k], 0));
            // every plan works in the same histogram and segment scratch: one at a time (plans
            // from the second chunk's on follow one another on their stream anyway)
            if (k == 1) HIP_CHECK(hipStreamWaitEvent(E.plan_stream, E.chunk_planned[0], 0));
            run_plan(E, chunks[k].first, chunks[k].second, E.plan_stream);
            HIP_CHECK(hipEventRecord(E.chunk_planned[k], E.plan_stream));
        };
        try {
            stage_steps(E, host, chunks[0].first, chunks[0].second);
            enqueue(0);
            for (size_t k = 0; k < chunks.size(); ++k) {
                if (k > 0) HIP_CHECK(hipStreamWaitEvent(st, E.chunk_planned[k], 0));
                if (k == 0) HIP_CHECK(hipEventRecord(E.ev[2], st));
                E.counts_known = readback && k > 0;
                if (E.counts_known) {  // waited for when the chunk's first update is due
                    E.counts_wait = E.chunk_planned[k];
                    E.counts_pending = true;
                }
                // the next chunk's upload and plan go out as soon as the helper has staged it, between
                // this chunk's step launches: the plan is a chain of short launches and needs the
                // time this chunk's kernels take
                bool next_out = k + 1 >= chunks.size();
                for (int i = chunks[k].first; i < chunks[k].first + chunks[k].second; ++i) {
                    run_step(E, i);
                    if (!next_out) {
                        std::unique_lock<std::mutex> lock(mu);
                        const bool staged_next = ready > k + 1;
                        lock.unlock();
                        if (staged_next) { enqueue(k + 1); next_out = true; }
                    }
                }
                done += chunks[k].second;
                if (!next_out) {
                    std::unique_lock<std::mutex> lock(mu);
                    cv.wait(lock, [&]() { return ready > k + 1 || failed; });
                    if (ready <= k + 1) std::rethrow_exception(failed);
                    lock.unlock();
                    enqueue(k + 1);
                }
            }
            if (helper.joinable()) helper.join();
        } catch (...) {
            // an index out of range in a later chunk: the chunks before it have run
            if (helper.joinable()) helper.join();
            (void)hipStreamSynchronize(E.copy_stream);
            (void)hipStreamSynchronize(E.plan_stream);
            (void)hipStreamSynchronize(st);
            E.step += (uint32_t)done;
            E.staged = false;
            throw;
        }
        E.staged = true;  // the whole batch is resident now
    }
    launch_loss_finalize(E.loss_part.p + (size_t)s0 * E.S * E.n_part, sn, E.S, E.n_part, 1.f / (float)sn,
                         E.d_loss_pin, st, E.reg_on ? E.reg_loss_part.p + (size_t)s0 * E.S : nullptr, E.loss_step.p);
    HIP_CHECK(hipGetLastError());
    HIP_CHECK(hipEventRecord(E.ev[3], st));
    HIP_CHECK(hipStreamSynchronize(st));
    std::memcpy(loss, E.h_loss_pin, S * 4);
    E.step += (uint32_t)sn;
    for (int k = 0; k < 3; ++k) HIP_CHECK(hipEventElapsedTime(&E.phase_ms[k], E.ev[k], E.ev[k + 1]));
    HIP_CHECK(hipEventElapsedTime(&E.phase_ms[3], E.ev[0], E.ev[3]));
    if (E.profile_kernels) collect_kernel_times(E);
}

void run_stage_batch(kge_engine& E, const Items& in) {
    const BatchPtrs b = bind_batch(E, in);
    E.staged = false;
    stage_steps(E, b, 0, E.n_step);
    upload_steps(E, 0, E.n_step, E.stream);
    HIP_CHECK(hipStreamSynchronize(E.stream));
    E.staged = true;
}

// "timing": phase_ms f32[4] {upload, plan, steps, total} of the last loop;
// kernel_ms f32[K_COUNT], kernel_calls u32[K_COUNT] accumulated since the last
// "timing" call (only with execution.profile_kernels); plan_counts
// u32[n_step, 4] {distinct entity rows, entity chunks, relation rows, relation chunks}.
void run_timing(kge_engine& E, const Items& in) {
    if (in.find("phase_ms")) {
        float* p = (float*)in.array("phase_ms", KGE_F32, {4});
        std::memcpy(p, E.phase_ms, sizeof(E.phase_ms));
    }
    if (in.find("kernel_ms")) {
        float* p = (float*)in.array("kernel_ms", KGE_F32, {(size_t)K_COUNT});
        uint32_t* c = (uint32_t*)in.array("kernel_calls", KGE_U32, {(size_t)K_COUNT});
        for (int k = 0; k < K_COUNT; ++k) {
            p[k] = (float)E.kernel_ms[k];
            c[k] = E.kernel_calls[k];
            E.kernel_ms[k] = 0;
            E.kernel_calls[k] = 0;
        }
    }
    if (in.find("plan_counts")) {
        uint32_t* p = (uint32_t*)in.array("plan_counts", KGE_U32, {(size_t)E.n_step, 4});
        std::vector<uint32_t> e(2 * E.n_step), r(2 * E.n_step);
        HIP_CHECK(hipMemcpy(e.data(), E.e_counts.p, e.size() * 4, hipMemcpyDeviceToHost));
        HIP_CHECK(hipMemcpy(r.data(), E.r_counts.p, r.size() * 4, hipMemcpyDeviceToHost));
        for (int i = 0; i < E.n_step; ++i) {
            p[4 * i + 0] = e[2 * i]; p[4 * i + 1] = e[2 * i + 1];
            p[4 * i + 2] = r[2 * i]; p[4 * i + 3] = r[2 * i + 1];
        }
    }
}

// "plan_dump": the index work of one step of the last train_step_loop call, as the device
// left it.  The plan phase is the device-side counterpart of the host's unique_pad
// (src/python/poplar_kge_dataset.py:161-164: distinct rows, inverse indices) and of the grouping
// multiUpdateAdd does for duplicate indices (src/pag/pag.cpp:721-743), so every array here has
// an exact integer answer.  Items: step (scalar, index into the call's batch) and outputs
//   contribution_row u32[R]      table row of every head / tail contribution
//   unique_rows u32[R], segment_start u32[R + 1], segment_contributions u32[R]
//                                distinct rows ascending, their first sorted position, how many
//                                of their members are gradient contributions (the others are the
//                                zero-gradient `remote` slots)
//   sorted_items u32[2 R]        item numbers in (row, item) order: item < R is contribution
//                                `item`, item >= R is slot `item - R` of `remote`
//   counts u32[2]                {distinct rows, chunks}
// and the same for the relation plan under relation_* (N = S B + n_relation items per copy);
//   label_column u32[S B]        the score column that holds every positive's label
//   tail_count u32[S], tail_column u32[S T], tail_multiplicity f32[S T]
//                                (merged tails) distinct tail rows per block, the column of every
//                                tail position, the positions every column stands for
void run_plan_dump(kge_engine& E, const Items& in) {
    const size_t i = in.uint("step");
    if (i >= (size_t)E.n_step || !E.e_sorted_vals) throw std::invalid_argument("'plan_dump' needs a planned step of the last train_step_loop");
    const size_t R = E.R, NRI = E.n_rel_items, RU = E.r_ustride;
    HIP_CHECK(hipStreamSynchronize(E.stream));
    auto out = [&](const char* name, const uint32_t* dev, size_t n) {
        if (!in.find(name)) return;
        uint32_t* host = (uint32_t*)in.array(name, KGE_U32, {n});
        HIP_CHECK(hipMemcpy(host, dev, n * 4, hipMemcpyDeviceToHost));
    };
    out("contribution_row", E.ckey.p + i * R, R);
    out("unique_rows", E.e_uniq.p + i * E.e_ustride, R);
    out("segment_start", E.e_seg.p + i * (E.e_ustride + 1), R + 1);
    out("segment_contributions", E.e_real.p + i * E.e_ustride, R);
    out("sorted_items", E.e_sorted_vals + i * 2 * R, 2 * R);
    out("counts", E.e_counts.p + 2 * i, 2);
    out("relation_unique_rows", E.r_uniq.p + i * RU, RU);
    out("relation_segment_start", E.r_seg.p + i * (RU + 1), RU + 1);
    out("relation_segment_contributions", E.r_real.p + i * RU, RU);
    out("relation_sorted_items", E.r_sorted_vals + i * NRI, NRI);
    out("relation_counts", E.r_counts.p + 2 * i, 2);
    out("label_column", E.clabel.p + i * (size_t)E.S * E.B, (size_t)E.S * E.B);
    // merged tails: distinct rows per block, the column of every tail position, and how many
    // positions every column stands for (float32, as the kernels read it)
    const size_t ST = (size_t)E.S * E.T;
    if (in.find("tail_count") || in.find("tail_column") || in.find("tail_multiplicity")) {
        if (!E.merge_tails) throw std::invalid_argument("'plan_dump': the tail lists were not merged (execution.merge_tails)");
        out("tail_count", E.tcount.p + i * E.S, E.S);
        out("tail_column", E.tcol.p + i * ST, ST);
        if (in.find("tail_multiplicity")) {
            float* host = (float*)in.array("tail_multiplicity", KGE_F32, {ST});
            HIP_CHECK(hipMemcpy(host, E.tmult.p + i * ST, ST * 4, hipMemcpyDeviceToHost));
        }
    }
}

// "grad_dump" (with execution.keep_gradients): the gradients the last step's updates were made
// from, as the step's loss.backward(lossScale) leaves them after multiUpdateAdd
// (src/poplar_kge.cpp:691, src/pag/pag.cpp:721-743), i.e. times the loss scale:
//   unique_rows u32[R], counts u32[2]   the step's distinct entity rows (ascending), how many
//   entity_gradient f32[R, D]           their summed gradients, in that order
//   relation_gradient f32[n_relation rows, D]  every relation row's (TransH: then the normals')
void run_grad_dump(kge_engine& E, const Items& in) {
    if (!E.keep_gradients || E.last_step < 0)
        throw std::invalid_argument("'grad_dump' needs execution.keep_gradients and a train_step_loop before it");
    const size_t R = E.R, i = (size_t)E.last_step;
    HIP_CHECK(hipStreamSynchronize(E.stream));
    if (in.find("unique_rows")) {
        uint32_t* host = (uint32_t*)in.array("unique_rows", KGE_U32, {R});
        HIP_CHECK(hipMemcpy(host, E.e_uniq.p + i * E.e_ustride, R * 4, hipMemcpyDeviceToHost));
    }
    if (in.find("counts")) {
        uint32_t* host = (uint32_t*)in.array("counts", KGE_U32, {2});
        HIP_CHECK(hipMemcpy(host, E.e_counts.p + 2 * i, 8, hipMemcpyDeviceToHost));
    }
    if (in.find("entity_gradient")) {
        float* host = (float*)in.array("entity_gradient", KGE_F32, {R, (size_t)E.D});
        HIP_CHECK(hipMemcpy2D(host, (size_t)E.D * 4, E.gkeep_e.p, (size_t)E.Dp * 4, (size_t)E.D * 4, R, hipMemcpyDeviceToHost));
    }
    if (in.find("relation_gradient")) {
        float* host = (float*)in.array("relation_gradient", KGE_F32, {(size_t)E.n_rel_rows, (size_t)E.D});
        HIP_CHECK(hipMemcpy2D(host, (size_t)E.D * 4, E.gkeep_r.p, (size_t)E.Dp * 4, (size_t)E.D * 4, (size_t)E.n_rel_rows,
                              hipMemcpyDeviceToHost));
    }
}

// "predict" (Model::predict, src/poplar_kge.cpp:811-855): for every (head row,
// relation) of every shard the n_best best-scoring tails of every shard's table.
//   predict_head, predict_relation  u32[S, Hb]   rows inside the query's own shard
//   predict_entity_count            u32[S]       real rows per shard (rows 1..count)
//   predict_scores  f32[S, S, Hb, n_best], predict_indices u32[S, S, Hb, n_best]:
//       [query shard, tail shard, query, rank], best first (ties: lower row first)
// Rows past the count never enter; when a shard has fewer than n_best rows the
// rest reads score -1e6, row 0 (the collector's initial content in the reference).
// With execution.shared_table the one table is scanned in S contiguous row
// ranges ("tail shards"), indices are table rows, the count is element 0.
void run_predict(kge_engine& E, const Items& in) {
    const size_t S = E.S, Hb = (size_t)E.predict_hr_batch, nb = (size_t)E.predict_n_best;
    if (nb < 1 || nb > 1024) throw std::invalid_argument("'execution.predict_n_best' must be in [1, 1024]");
    const uint32_t* head = (const uint32_t*)in.array("predict_head", KGE_U32, {S, Hb});
    const uint32_t* relation = (const uint32_t*)in.array("predict_relation", KGE_U32, {S, Hb});
    const uint32_t* count = (const uint32_t*)in.array("predict_entity_count", KGE_U32, {S});
    float* out_s = (float*)in.array("predict_scores", KGE_F32, {S, S, Hb, nb});
    uint32_t* out_i = (uint32_t*)in.array("predict_indices", KGE_U32, {S, S, Hb, nb});
    const hipStream_t st = E.stream;
    const int Q = (int)(S * Hb), Qp = round_up(Q, 128), Dp = E.Dp;
    // Default: 2^25 scores per launch (262144 tails for 128 queries; 400 MB for the three score
    // buffers): the events between the two streams cost about 10 us per launch, measured 19.3 /
    // 16.2 / 15.6 ms for a 22.8M-row sweep with 65536 / 131072 / 262144 tails per launch.
    const int auto_rows = std::clamp((1 << 25) / Qp / 1024 * 1024, 8192, 262144);
    const int chunk = round_up((int)std::min<int64_t>(E.n_entity, E.predict_chunk_rows ? E.predict_chunk_rows : auto_rows), 64);

    std::vector<uint32_t> rows(Qp, 0u), rels(Qp, 0u);
    for (size_t s = 0; s < S; ++s) {
        if (count[s] >= (uint32_t)E.n_entity)
            throw std::invalid_argument("'predict_entity_count' must be < model.n_entity (row 0 is padding)");
        for (size_t j = 0; j < Hb; ++j) {
            const uint32_t h = head[s * Hb + j], r = relation[s * Hb + j];
            if (h >= (uint32_t)E.n_entity) throw std::invalid_argument("'predict_head' index out of range");
            if (r >= (uint32_t)E.n_rel) throw std::invalid_argument("'predict_relation' index out of range");
            rows[s * Hb + j] = (E.shared_table ? 0u : (uint32_t)s * (uint32_t)E.n_entity) + h;
            rels[s * Hb + j] = r;
        }
    }
    if (E.p_idx.n < (size_t)(Qp + chunk)) {
        E.p_idx.alloc(Qp + chunk);
        E.p_rel.alloc(Qp);
        E.p_count.alloc(2);
        E.p_opnd.alloc((size_t)(Qp + chunk) * Dp);
        E.p_scores.alloc((size_t)kge_engine::kScoreBuffers * Qp * chunk);  // chunks being merged and being scored
        if (E.score_fn == SCORE_TRANSH) {
            E.p_opnd_n.alloc((size_t)(Qp + chunk) * Dp);
            E.p_cmat.alloc((size_t)Qp * chunk);
        }
        E.p_best_s.alloc((size_t)Q * nb);
        E.p_best_i.alloc((size_t)Q * nb);
        if (E.F) {
            E.p_hidden.alloc((size_t)std::max(Qp, chunk) * Dp);
            E.p_featd.alloc((size_t)std::max(Qp, chunk) * E.Fp);
            if (E.mlp) {
                E.p_fproj.alloc((size_t)std::max(Qp, chunk) * Dp);
                E.p_concat.alloc((size_t)std::max(Qp, chunk) * 2 * Dp);
                E.p_pre.alloc((size_t)std::max(Qp, chunk) * E.mlp);
            }
        }
    }
    const size_t pin_need = (size_t)Qp * 8 + (size_t)Q * nb * 8;
    if (E.p_pin_bytes < pin_need) {
        if (E.p_pin) HIP_CHECK(hipHostFree(E.p_pin));
        E.p_pin = nullptr; E.p_pin_bytes = 0;
        HIP_CHECK(hipHostMalloc(&E.p_pin, pin_need, hipHostMallocDefault));
        E.p_pin_bytes = pin_need;
    }
    uint32_t* pin_rows = (uint32_t*)E.p_pin;
    uint32_t* pin_rels = pin_rows + Qp;
    float* got_s = (float*)(pin_rels + Qp);
    uint32_t* got_i = (uint32_t*)(got_s + (size_t)Q * nb);
    std::memcpy(pin_rows, rows.data(), (size_t)Qp * 4);
    std::memcpy(pin_rels, rels.data(), (size_t)Qp * 4);
    HIP_CHECK(hipMemcpyAsync(E.p_idx.p, pin_rows, (size_t)Qp * 4, hipMemcpyHostToDevice, st));
    HIP_CHECK(hipMemcpyAsync(E.p_rel.p, pin_rels, (size_t)Qp * 4, hipMemcpyHostToDevice, st));

    if (E.F) {  // the two row counts of this call's feature products (queries, a chunk of tails), uploaded once
        const uint32_t counts[2] = {(uint32_t)Qp, (uint32_t)chunk};
        HIP_CHECK(hipMemcpy(E.p_count.p, counts, sizeof(counts), hipMemcpyHostToDevice));
    }
    // rows `idx[0..n)` of the table as a row source: the embeddings, or hidden = emb + feature . W
    // (`net`: the head's feature network for the queries, the tail's for the candidates)
    auto rows_of = [&](const uint32_t* idx, int n, int net) {
        RowSource r;
        r.base = E.table.p; r.pitch = E.L.pitch; r.etype = E.L.emb_etype;
        r.index = idx; r.count = Dp; r.vec = 1;
        if (E.F) {
            // the row count as the feature kernels read it: one of the call's two constants
            const uint32_t* count = E.p_count.p + (n == Qp ? 0 : 1);
            FeatureArgs fa = {};
            fa.uniq_key = idx; fa.counts = count; fa.max_rows = n;
            fa.emb_base = E.table.p; fa.feat_base = E.table.p + E.L.off_f; fa.pitch = E.L.pitch;
            fa.emb_etype = E.L.emb_etype; fa.feat_etype = E.L.feat_etype;
            fa.Dp = Dp; fa.Fp = E.Fp; fa.proj = E.proj.p + (size_t)net * E.Fp * Dp;
            fa.featd = E.p_featd.p; fa.use_mfma = E.use_mfma;
            if (E.mlp) {
                FeatureArgs fp = fa;
                fp.emb_base = nullptr;
                launch_hidden_fwd(fp, E.p_fproj.p, st);
                MlpArgs ma = {};
                ma.uniq_key = idx; ma.counts = count; ma.max_rows = n;
                ma.emb_base = E.table.p; ma.pitch = E.L.pitch; ma.emb_etype = E.L.emb_etype;
                ma.Dp = Dp; ma.M = E.mlp;
                ma.up = E.up.p + (size_t)net * 2 * Dp * E.mlp; ma.down = E.down.p + (size_t)net * E.mlp * Dp;
                ma.concat = E.p_concat.p; ma.pre = E.p_pre.p; ma.add_value = 1;
                launch_mlp_fwd(ma, E.p_fproj.p, E.p_hidden.p, st);
            } else
            launch_hidden_fwd(fa, E.p_hidden.p, st);
            r.base = (const char*)E.p_hidden.p; r.pitch = (int64_t)Dp * 4; r.etype = ET_F32; r.index = nullptr;
        }
        return r;
    };
    // predicted tails of all queries: dense rows [0, Qp)
    launch_gather_operands(rows_of(E.p_idx.p, Qp, 0), E.rel.p, E.p_rel.p, rel_mode_of(E), E.D / 2, Qp,
                           Qp, Dp, E.p_opnd.p, nullptr, st);

    const bool transh = E.score_fn == SCORE_TRANSH;
    if (transh) {  // unit normals beside the predicted tails (transHPredict, :539-549)
        HIP_CHECK(hipMemcpyAsync(E.p_opnd_n.p, E.p_opnd.p, (size_t)Qp * Dp * 4, hipMemcpyDeviceToDevice, st));
        launch_transh_predict(E.rel.p, E.p_rel.p, E.n_rel, Qp, Dp, E.p_opnd.p, E.p_opnd_n.p, st);
    }

    ScoreShape sh = {};
    sh.S = 1; sh.B = Qp; sh.T = chunk; sh.Dp = Dp;
    sh.score_fn = E.score_fn; sh.dist_fn = E.dist_fn; sh.loss_fn = E.loss_fn;
    sh.gamma = E.gamma; sh.loss_scale = 1.f; sh.use_mfma = E.use_mfma; sh.operands_dense = 1;
    RowSource dense;
    dense.base = (const char*)E.p_opnd.p; dense.pitch = (int64_t)Dp * 4; dense.etype = ET_F32;
    dense.index = nullptr; dense.count = Dp; dense.vec = 1;
    RowSource dense_n = dense;
    dense_n.base = (const char*)E.p_opnd_n.p;
    ScoreShape dot = sh;
    dot.score_fn = SCORE_DISTMULT; dot.dist_fn = DIST_DOT;

    const float init_score = -1e6f;
    uint32_t init_bits;
    std::memcpy(&init_bits, &init_score, 4);
    const int64_t per_range = ((int64_t)E.n_entity - 1 + (int64_t)S - 1) / (int64_t)S;
    const hipStream_t mst = E.merge_stream;
    const size_t score_elems = (size_t)Qp * chunk;
    for (size_t ts = 0; ts < S; ++ts) {
        // the n_best lists belong to the merge stream (the previous tail shard's read-back waited for it)
        launch_fill_u32((uint32_t*)E.p_best_s.p, init_bits, (int64_t)(Q * nb), mst);
        launch_fill_u32(E.p_best_i.p, 0u, (int64_t)(Q * nb), mst);
        int64_t lo, hi, table_off;
        if (E.shared_table) {
            lo = 1 + (int64_t)ts * per_range;
            hi = std::min<int64_t>(lo + per_range, 1 + (int64_t)count[0]);
            table_off = 0;
        } else {
            lo = 1; hi = 1 + (int64_t)count[ts]; table_off = (int64_t)ts * E.n_entity;
        }
        int64_t n_chunk = 0;
        for (int64_t r0 = lo; r0 < hi; r0 += chunk, ++n_chunk) {
            const int live = (int)std::min<int64_t>(chunk, hi - r0);
            const int buf = (int)(n_chunk % kge_engine::kScoreBuffers);
            float* scores = E.p_scores.p + (size_t)buf * score_elems;
            uint32_t* tail_idx = E.p_idx.p + Qp;
            // Consecutive table rows need no row list, and most are scored where they lie (the tails
            // take no relation): the kernels take whole tiles of 64 rows, so a chunk's last tile may
            // read up to 63 rows past the shard's count - rows of the table all the same (it ends in
            // kSpareRows rows that belong to nobody), whose scores the merge never looks at.
            // TransH's two operand matrices go through the dense copy, and so do 16-bit rows on the
            // matrix-core kernels (their fast staging path takes float32 rows, and converting while
            // copying costs less than the slower path does).
            const int live_tiles = round_up(live, 64);
            const bool in_place = !E.F && !transh &&
                                  (E.L.emb_etype == ET_F32 || !E.use_mfma || (E.dist_fn == DIST_L1 && E.score_fn != SCORE_DISTMULT));
            const int n_tail = in_place ? live_tiles : chunk;  // rows the scoring launch covers = the scores' row pitch
            RowSource tails;
            if (!E.F && (in_place || live == chunk)) {
                tails.base = E.table.p + (table_off + r0) * E.L.pitch; tails.pitch = E.L.pitch;
                tails.etype = E.L.emb_etype; tails.index = nullptr; tails.count = Dp; tails.vec = 1;
            } else {
                launch_row_range((uint32_t)(table_off + r0), live, chunk, tail_idx, st);
                tails = rows_of(tail_idx, chunk, E.nets - 1);
            }
            if (!in_place)
                launch_gather_operands(tails, E.rel.p, nullptr, 0, 0, 0, chunk, Dp, E.p_opnd.p + (size_t)Qp * Dp, nullptr, st);
            // this buffer's previous scores must have been merged
            if (n_chunk >= kge_engine::kScoreBuffers) HIP_CHECK(hipStreamWaitEvent(st, E.merged[buf], 0));
            if (in_place) {
                ScoreShape shp = sh;
                shp.T = n_tail;
                launch_score_fwd_rows(shp, dense, tails, scores, st);
            }
            else
            if (transh) {  // transHScore (:551-565): c = n . tail, then the L1 part
                HIP_CHECK(hipMemcpyAsync(E.p_opnd_n.p + (size_t)Qp * Dp, E.p_opnd.p + (size_t)Qp * Dp,
                                         (size_t)chunk * Dp * 4, hipMemcpyDeviceToDevice, st));
                launch_score_fwd(dot, dense_n, E.rel.p, nullptr, nullptr, E.p_cmat.p, nullptr, nullptr, nullptr,
                                 false, st);
                TranshFwd tf;
                tf.sh = sh; tf.pt = E.p_opnd.p; tf.nt = E.p_opnd_n.p; tf.cmat = E.p_cmat.p; tf.clabel = nullptr;
                tf.coef = scores; tf.dcm = nullptr; tf.loss_part = nullptr;
                launch_transh_fwd(tf, false, st);
            } else
            launch_score_fwd(sh, dense, E.rel.p, nullptr, nullptr, scores, nullptr, nullptr, nullptr,
                             false, st);
            HIP_CHECK(hipEventRecord(E.scored[buf], st));
            HIP_CHECK(hipStreamWaitEvent(mst, E.scored[buf], 0));
            launch_topk_merge(scores, n_tail, Q, live, (uint32_t)r0, (int)nb, E.p_best_s.p, E.p_best_i.p, mst);
            HIP_CHECK(hipEventRecord(E.merged[buf], mst));
        }
        HIP_CHECK(hipGetLastError());
        HIP_CHECK(hipMemcpyAsync(got_s, E.p_best_s.p, (size_t)Q * nb * 4, hipMemcpyDeviceToHost, mst));
        HIP_CHECK(hipMemcpyAsync(got_i, E.p_best_i.p, (size_t)Q * nb * 4, hipMemcpyDeviceToHost, mst));
        HIP_CHECK(hipStreamSynchronize(mst));
        HIP_CHECK(hipStreamSynchronize(st));
        for (size_t hs = 0; hs < S; ++hs) {
            std::memcpy(out_s + (hs * S + ts) * Hb * nb, got_s + hs * Hb * nb, Hb * nb * 4);
            std::memcpy(out_i + (hs * S + ts) * Hb * nb, got_i + hs * Hb * nb, Hb * nb * 4);
        }
    }
}

// "gather_benchmark": the stand-alone row gather (fr::Buffer::read) over the
// engine's own table: gathers `indices` u32[n] physical rows `repeats` times
// into a scratch buffer and reports the mean kernel time in `ms` f32[1].
void run_gather_benchmark(kge_engine& E, const Items& in) {
    const kge_item& idx = in.typed("indices", KGE_U32);
    if (idx.rank != 1) throw std::invalid_argument("'indices' expected a 1-D array");
    const size_t n = idx.shape[0];
    float* ms = (float*)in.array("ms", KGE_F32, {1});
    const unsigned repeats = in.find("repeats") ? in.uint("repeats") : 10u;
    const uint32_t* h = (const uint32_t*)idx.data;
    for (size_t i = 0; i < n; ++i)
        if ((int64_t)h[i] >= E.n_rows) throw std::invalid_argument("'indices' out of range");
    DevBuf<uint32_t> d_idx;
    DevBuf<char> out;
    d_idx.alloc(n);
    out.alloc(n * (size_t)E.L.pitch);
    HIP_CHECK(hipMemcpy(d_idx.p, h, n * 4, hipMemcpyHostToDevice));
    launch_rows_gather(E.table.p, d_idx.p, out.p, (int64_t)n, E.L.pitch, E.stream);
    HIP_CHECK(hipEventRecord(E.ev[0], E.stream));
    for (unsigned r = 0; r < repeats; ++r)
        launch_rows_gather(E.table.p, d_idx.p, out.p, (int64_t)n, E.L.pitch, E.stream);
    HIP_CHECK(hipEventRecord(E.ev[1], E.stream));
    HIP_CHECK(hipStreamSynchronize(E.stream));
    float t = 0.f;
    HIP_CHECK(hipEventElapsedTime(&t, E.ev[0], E.ev[1]));
    ms[0] = t / (float)repeats;
}

void set_error(char* err, size_t len, const char* what) {
    if (err && len) {
        std::strncpy(err, what, len - 1);
        err[len - 1] = 0;
    }
}

template <class Fn>
int guarded(char* err, size_t len, Fn&& fn) {
    try {
        fn();
        return KGE_OK;
    } catch (const std::invalid_argument& e) {
        set_error(err, len, e.what());
        return KGE_INVALID_ARGUMENT;
    } catch (const std::logic_error& e) {
        set_error(err, len, e.what());
        return KGE_LOGIC_ERROR;
    } catch (const std::exception& e) {
        set_error(err, len, e.what());
        return KGE_RUNTIME_ERROR;
    }
}

}  // namespace

extern "C" {

int kge_engine_create(const kge_item* settings, size_t n_settings, const char* gp_folder,
                      kge_engine** out, char* err, size_t err_len) {
    (void)gp_folder;
    return guarded(err, err_len, [&] {
        if (!out) throw std::invalid_argument("null output pointer");
        std::unique_ptr<kge_engine> E(new kge_engine());
        parse_settings(*E, Items{settings, n_settings});
        allocate(*E);
        *out = E.release();
    });
}

int kge_engine_run(kge_engine* engine, const char* command, kge_item* items, size_t n_items,
                   char* err, size_t err_len) {
    return guarded(err, err_len, [&] {
        if (!engine || !command) throw std::invalid_argument("null engine or command");
        kge_engine& E = *engine;
        const Items in{items, n_items};
        const std::string cmd = command;
        if (cmd == "train_step_loop") run_train_step_loop(E, in);
        else if (cmd == "read_entity") run_read_entity(E, in);
        else if (cmd == "write_entity") run_write_entity(E, in, false);
        else if (cmd == "write_entity_raw") run_write_entity(E, in, true);
        else if (cmd == "read") run_read_write(E, false, in);
        else if (cmd == "write") run_read_write(E, true, in);
        else if (cmd == "stage_batch") run_stage_batch(E, in);
        else if (cmd == "timing") run_timing(E, in);
        else if (cmd == "plan_dump") run_plan_dump(E, in);
        else if (cmd == "grad_dump") run_grad_dump(E, in);
        else if (cmd == "gather_benchmark") run_gather_benchmark(E, in);
        else if (cmd == "variables") { /* served by kge_engine_variable_info */ }
        else if (cmd == "predict") run_predict(E, in);
        else
            throw std::invalid_argument("Unknown command '" + cmd + "'");
    });
}

size_t kge_engine_variable_count(const kge_engine* engine) { return engine ? engine->variables.size() : 0; }

int kge_engine_variable_info(const kge_engine* engine, size_t index, const char** name,
                             const size_t** shape, size_t* rank) {
    if (!engine || index >= engine->variables.size()) return KGE_INVALID_ARGUMENT;
    const Variable& v = engine->variables[index];
    *name = v.name.c_str();
    *shape = v.shape.data();
    *rank = v.shape.size();
    return KGE_OK;
}

void kge_engine_destroy(kge_engine* engine) {
    if (!engine) return;
    if (engine->stream) (void)hipStreamSynchronize(engine->stream);
    delete engine;
}

// ---- device ops --------------------------------------------------------------

static int op_status(const char* what) {
    (void)what;
    return hipGetLastError() == hipSuccess ? KGE_OK : KGE_RUNTIME_ERROR;
}

static bool bad_dims(int M, int N, int D) { return M < 0 || N < 0 || D < 1; }

int kge_l1_distance(const float* a, const float* b, float* out, int M, int N, int D, void* stream) {
    if (bad_dims(M, N, D)) return KGE_INVALID_ARGUMENT;
    if (M == 0 || N == 0) return KGE_OK;
    launch_distance(DIST_L1, a, b, out, M, N, D, (hipStream_t)stream);
    return op_status("l1_distance");
}
int kge_l2_distance(const float* a, const float* b, float* out, int M, int N, int D, void* stream) {
    if (bad_dims(M, N, D)) return KGE_INVALID_ARGUMENT;
    if (M == 0 || N == 0) return KGE_OK;
    launch_distance(DIST_L2, a, b, out, M, N, D, (hipStream_t)stream);
    return op_status("l2_distance");
}
int kge_dot_score(const float* a, const float* b, float* out, int M, int N, int D, void* stream) {
    if (bad_dims(M, N, D)) return KGE_INVALID_ARGUMENT;
    if (M == 0 || N == 0) return KGE_OK;
    launch_distance(DIST_DOT, a, b, out, M, N, D, (hipStream_t)stream);
    return op_status("dot_score");
}
int kge_l1_distance_grad(const float* a, const float* b, const float* g, float* grad, int M, int N,
                         int D, void* stream) {
    if (bad_dims(M, N, D)) return KGE_INVALID_ARGUMENT;
    if (M == 0) return KGE_OK;
    launch_distance_grad(DIST_L1, a, b, nullptr, g, grad, M, N, D, (hipStream_t)stream);
    return op_status("l1_distance_grad");
}
int kge_l2_distance_grad(const float* a, const float* b, const float* dist, const float* g,
                         float* grad, int M, int N, int D, void* stream) {
    if (bad_dims(M, N, D)) return KGE_INVALID_ARGUMENT;
    if (M == 0) return KGE_OK;
    launch_distance_grad(DIST_L2, a, b, dist, g, grad, M, N, D, (hipStream_t)stream);
    return op_status("l2_distance_grad");
}
int kge_buffer_read(const void* buf, const uint32_t* idx, void* out, int64_t n, int64_t row_bytes,
                    void* stream) {
    if (n < 0 || row_bytes < 4 || row_bytes % 4) return KGE_INVALID_ARGUMENT;
    launch_rows_gather(buf, idx, out, n, row_bytes, (hipStream_t)stream);
    return op_status("buffer_read");
}
int kge_buffer_write(void* buf, const uint32_t* idx, const void* data, int64_t n, int64_t row_bytes,
                     void* stream) {
    if (n < 0 || row_bytes < 4 || row_bytes % 4) return KGE_INVALID_ARGUMENT;
    launch_rows_scatter(buf, idx, data, n, row_bytes, (hipStream_t)stream);
    return op_status("buffer_write");
}

int kge_log_sigmoid(const float* x, const float* dy, float* y, float* dx, int64_t n, int form, void* stream) {
    if (n < 0 || (form != 0 && form != 1) || (n > 0 && !x)) return KGE_INVALID_ARGUMENT;
    launch_log_sigmoid(x, dy, y, dx, n, form, (hipStream_t)stream);
    return op_status("log_sigmoid");
}
int kge_log_softmax(const float* x, float* y, int64_t rows, int64_t cols, void* stream) {
    if (rows < 0 || cols < 1 || (rows > 0 && (!x || !y))) return KGE_INVALID_ARGUMENT;
    launch_log_softmax(x, nullptr, y, rows, cols, (hipStream_t)stream);
    return op_status("log_softmax");
}
int kge_log_softmax_grad(const float* y, const float* dy, float* dx, int64_t rows, int64_t cols, void* stream) {
    if (rows < 0 || cols < 1 || (rows > 0 && (!y || !dy || !dx))) return KGE_INVALID_ARGUMENT;
    launch_log_softmax(y, dy, dx, rows, cols, (hipStream_t)stream);
    return op_status("log_softmax_grad");
}
int kge_loss(int loss_fn, const float* score, const uint32_t* label, int S, int B, int T,
             float softmax_correction, float negative_adversarial_scale, float loss_scale,
             float* loss, float* row_loss, float* dscore, void* stream) {
    if ((loss_fn != LOSS_LOGSIGMOID && loss_fn != LOSS_SOFTMAX) || S < 1 || B < 1 || T < 2) return KGE_INVALID_ARGUMENT;
    if (!score || !label || !loss || !row_loss || !dscore) return KGE_INVALID_ARGUMENT;
    const hipStream_t st = (hipStream_t)stream;
    ScoreShape sh = {};
    sh.S = S; sh.B = B; sh.T = T; sh.Dp = 0;
    // a score that is the distance function's value itself: the coefficient launch_loss_rows
    // leaves is d loss / d score (times the loss scale), without the sign of gamma - distance
    sh.score_fn = SCORE_DISTMULT; sh.dist_fn = DIST_DOT; sh.loss_fn = loss_fn;
    sh.loss_scale = loss_scale; sh.softmax_correction = softmax_correction;
    sh.negative_adversarial_scale = negative_adversarial_scale;
    if (dscore != score &&
        hipMemcpyAsync(dscore, score, (size_t)S * B * T * 4, hipMemcpyDeviceToDevice, st) != hipSuccess)
        return KGE_RUNTIME_ERROR;
    launch_loss_rows(sh, label, dscore, nullptr, row_loss, nullptr, st);
    launch_loss_finalize(row_loss, 1, S, B, 1.f, loss, st);
    return op_status("loss");
}

namespace {
struct ScatterLayout {
    size_t N, tiles, cmax;
    size_t off_keys_a, off_vals_a, off_keys_b, off_vals_b, off_hist, off_uniq, off_seg, off_coff,
        off_cpos, off_clen, off_counts, off_real, off_scratch, off_partial, total;
};
ScatterLayout scatter_layout(int64_t n, int64_t rows, int64_t cols) {
    ScatterLayout L;
    L.N = (size_t)(n + rows);
    L.tiles = (L.N + kSortTile - 1) / kSortTile;
    L.cmax = (size_t)rows + (size_t)n / 32 + 1;
    size_t o = 0;
    auto take = [&](size_t words) { size_t at = o; o += (words * 4 + 15) / 16 * 16; return at; };
    L.off_keys_a = take(L.N); L.off_vals_a = take(L.N);
    L.off_keys_b = take(L.N); L.off_vals_b = take(L.N);
    L.off_hist = take(radix_sort_hist_words((int)L.N, 1, std::max(1, bit_length((uint64_t)rows - 1)) + kKeyFlagBits));
    L.off_uniq = take(rows); L.off_seg = take(rows + 1); L.off_coff = take(rows + 1);
    L.off_cpos = take(L.cmax); L.off_clen = take(L.cmax); L.off_counts = take(2);
    L.off_real = take(rows); L.off_scratch = take(find_segments_scratch_words((int)L.N, 0, 1));
    L.off_partial = take(L.cmax * (size_t)cols);
    L.total = o;
    return L;
}
}  // namespace

size_t kge_scatter_add_workspace_bytes(int64_t n, int64_t rows, int64_t cols) {
    if (n < 0 || rows < 1 || cols < 1) return 0;
    return scatter_layout(n, rows, cols).total;
}

int kge_scatter_add(float* grad_t, int64_t rows, int64_t cols, const uint32_t* idx, int64_t n,
                    const float* grad_out, void* workspace, void* stream) {
    if (n < 0 || rows < 1 || cols < 1 || n + rows >= ((int64_t)1 << 31)) return KGE_INVALID_ARGUMENT;
    if (!workspace || (uintptr_t)workspace % 16) return KGE_INVALID_ARGUMENT;
    const hipStream_t st = (hipStream_t)stream;
    const ScatterLayout L = scatter_layout(n, rows, cols);
    char* w = (char*)workspace;
    auto u32 = [&](size_t off) { return (uint32_t*)(w + off); };
    launch_iota_keys(idx, u32(L.off_keys_a), u32(L.off_vals_a), n, rows, st);
    const int bits = std::max(1, bit_length((uint64_t)rows - 1)) + kKeyFlagBits;
    const int which = launch_radix_sort(u32(L.off_keys_a), u32(L.off_vals_a), u32(L.off_keys_b),
                                        u32(L.off_vals_b), u32(L.off_hist), (int)L.N, 1, bits, st);
    const uint32_t* sv = which ? u32(L.off_vals_b) : u32(L.off_vals_a);
    SegJob job = {};
    job.keys = which ? u32(L.off_keys_b) : u32(L.off_keys_a); job.vals = sv;
    job.N = (int)L.N; job.n_real = (int)n; job.chunk = 32; job.direct_max = 0;
    SegPlan& sp = job.plan;
    sp.uniq_key = u32(L.off_uniq); sp.seg_start = u32(L.off_seg); sp.chunk_off = u32(L.off_coff);
    sp.chunk_pos = u32(L.off_cpos); sp.chunk_len = u32(L.off_clen); sp.counts = u32(L.off_counts);
    sp.item_row = nullptr; sp.u_stride = (int)rows; sp.c_stride = (int)L.cmax;
    sp.seg_real = u32(L.off_real); sp.hot_rows = nullptr; sp.hot_count = nullptr; sp.host_counts = nullptr;
    launch_find_segments2(job, nullptr, 1, u32(L.off_scratch), st);
    ReduceArgs ra = {};
    ra.src.sorted_item = sv; ra.src.grad = grad_out; ra.src.transform = 0;
    ra.chunk_pos = sp.chunk_pos; ra.chunk_len = sp.chunk_len; ra.counts = sp.counts;
    ra.max_chunks = (int)L.cmax; ra.chunk = 32; ra.partial = (float*)(w + L.off_partial);
    ra.Dp = (int)cols;
    launch_reduce_chunks(ra, st);
    launch_sum_partials_rows(sp.chunk_off, ra.partial, rows, cols, grad_t, st);
    return op_status("scatter_add");
}

// ---- the scatter-add without a workspace argument and without allocation ----
// Callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc) get the workspace from a fixed array in device memory.  Each GPU holds its own
// copy of the array at its own address, which hipGetSymbolAddress reports with that GPU current:
// the address is looked up once per device and every later use goes through it (the array's name
// is a host-side stand-in in host code, not a device address).
}  // extern "C"

namespace {
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// the current device's copy of `scratch`, or null with `what` set
void* static_scratch(std::string& what) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        what = std::string("no current HIP device (") + (e != hipSuccess ? hipGetErrorString(e) : "index out of range") + ")";
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            (void)hipGetLastError();
            what = std::string("hipGetSymbolAddress(scratch) failed: ") + hipGetErrorString(e);
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" {

size_t kge_scatter_add_static_max_bytes(void) { return kStaticScratchBytes; }

int kge_scatter_add_static(float* grad_t, int64_t rows, int64_t cols, const uint32_t* idx, int64_t n,
                           const float* grad_out, void* stream, char* err, size_t err_len) {
    if (n < 0 || rows < 1 || cols < 1 || n + rows >= ((int64_t)1 << 31)) {
        set_error(err, err_len, "kge_scatter_add_static: sizes out of range (n >= 0, rows >= 1, cols >= 1, n + rows < 2^31)");
        return KGE_INVALID_ARGUMENT;
    }
    const size_t need = scatter_layout(n, rows, cols).total;
    if (need > kStaticScratchBytes) {
        std::ostringstream msg;
        msg << "kge_scatter_add_static: n = " << n << ", rows = " << rows << ", cols = " << cols << " need " << need
            << " bytes of workspace, more than the " << kStaticScratchBytes
            << " bytes of the static scratch array; use kge_scatter_add with a workspace of your own";
        set_error(err, err_len, msg.str().c_str());
        return KGE_INVALID_ARGUMENT;
    }
    std::string what;
    void* ptr = static_scratch(what);
    if (!ptr) {
        set_error(err, err_len, what.c_str());
        return KGE_RUNTIME_ERROR;
    }
    // nothing in the workspace has to start at zero: every word a kernel reads, an earlier kernel
    // of the same call wrote (histograms, keys, segment tables, partial sums)
    const int rc = kge_scatter_add(grad_t, rows, cols, idx, n, grad_out, ptr, stream);
    if (rc != KGE_OK) set_error(err, err_len, "kge_scatter_add_static: kernel launch failed");
    return rc;
}

int kge_adam(float* p, float* m, float* v, const float* g, int64_t n, float alpha, float beta_m,
             float beta_v, float epsilon, float weight_decay, int v_is_sqrt, void* stream) {
    if (n < 0) return KGE_INVALID_ARGUMENT;
    launch_adam_flat(p, m, v, g, n, alpha, beta_m, beta_v, epsilon, weight_decay, v_is_sqrt,
                     (hipStream_t)stream);
    return op_status("adam");
}

}  // extern "C"
