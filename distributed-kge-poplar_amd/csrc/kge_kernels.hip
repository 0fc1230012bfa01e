// gfx950 (CDNA4, wave64) kernels of the per-shard KGE training step.
//
// Reference semantics, by kernel:
//   build_items / radix sort / find_segments  host np.unique + multiUpdateAdd grouping
//       (src/python/poplar_kge_dataset.py:161-164, src/pag/pag.cpp:721-743)
//   score_fwd      predictTail + score + logsigmoid loss (src/poplar_kge.cpp:488-499,
//                  567-573, 615-636; l1/l2distance codelets)
//   loss_rows      softmax / adversarial loss (src/poplar_kge.cpp:623-652)
//   score_bwd      l1/l2distancegrad, matMul backward (src/pag/pag.cpp:685-700, 777-836)
//   reduce_chunks + adam_rows   multiUpdateAdd + fr::nn::adam + Buffer::write
//                  (src/fructose/frnn.cpp:61-90, src/poplar_kge.cpp:695-704)
#include "kge_device.h"

#include <algorithm>
#include <cstdint>
#include <stdexcept>
#include <type_traits>

namespace kge {

// --------------------------------------------------------------------------
// operand gather: one wave per contribution copies its entity (or hidden) row,
// converted to float32 and with the relation already applied for the heads
// (predicted tail h + r, or h * r), into the dense operand matrix the scoring
// kernels read: rows [0, n_head) = a-operands, the rest = b-operands.
// XF: the complex-product / rotation modes (3, 4) are compiled in (their code costs the
// plain modes registers otherwise)
template <bool XF>
__global__ __launch_bounds__(256) void k_gather_operands(RowSource ent, const float* __restrict__ rel,
                                                         const uint32_t* __restrict__ crel,
                                                         int rel_mode, int half, int n_head, int n_rows,
                                                         int Dp, float* __restrict__ out,
                                                         uint16_t* __restrict__ out16, TailCols tc) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (c >= n_rows || !tc.live(c - n_head)) return;
    const char* row = row_ptr(ent, c);
    const float* rrow = (c < n_head && rel_mode) ? rel + (size_t)crel[c] * Dp : nullptr;
    for (int k = lane * 4; k < Dp; k += 256) {
        float4 v = load4(row, k, ent);
        if (XF && rrow && rel_mode == 3) {
            // complex product: column kk pairs with kk +- half (src/poplar_kge.cpp:501-510)
            float* vv = &v.x;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int kk = k + x;
                if (kk >= 2 * half) { vv[x] = 0.f; continue; }
                const int pp = kk < half ? kk + half : kk - half;
                const float e2 = load1(row, pp, ent.etype);
                vv[x] = kk < half ? vv[x] * rrow[kk] - e2 * rrow[pp]    // re = h_re r_re - h_im r_im
                                  : e2 * rrow[kk] + vv[x] * rrow[pp];   // im = h_re r_im + h_im r_re
            }
        } else if (XF && rrow && rel_mode == 4) {
            // rotation by the relation's phases (src/poplar_kge.cpp:516-530): phase, sine and
            // cosine in float16, the rotation itself in float32
            float* vv = &v.x;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int kk = k + x;
                if (kk >= 2 * half) { vv[x] = 0.f; continue; }
                const int kq = kk < half ? kk : kk - half, pp = kk < half ? kk + half : kk - half;
                const float th = (float)(_Float16)rrow[kq];
                const float sn = (float)(_Float16)sinf(th), cs = (float)(_Float16)cosf(th);
                const float e2 = load1(row, pp, ent.etype);
                vv[x] = kk < half ? vv[x] * cs - e2 * sn     // re = h_re cos - h_im sin
                                  : vv[x] * cs + e2 * sn;    // im = h_im cos + h_re sin
            }
        } else if (rrow) v = combine_rel(v, rrow, k, rel_mode);
        // + 0 turns a -0 into +0, so that a difference of stored operands is never -0
        // (the paired L1 backward reads the sign off the difference's bit pattern)
        v.x += 0.f; v.y += 0.f; v.z += 0.f; v.w += 0.f;
        if (out16) {
            // bfloat16 scoring: the operands are rounded once, here; the float32 copy holds
            // the same rounded values, so every scoring kernel computes the same products
            const uint16_t h0 = f32_to_bf16(v.x), h1 = f32_to_bf16(v.y), h2 = f32_to_bf16(v.z), h3 = f32_to_bf16(v.w);
            uint2 raw;
            raw.x = (uint32_t)h0 | ((uint32_t)h1 << 16);
            raw.y = (uint32_t)h2 | ((uint32_t)h3 << 16);
            *reinterpret_cast<uint2*>(out16 + (size_t)c * Dp + k) = raw;
            v = make_float4(bf16_to_f32(h0), bf16_to_f32(h1), bf16_to_f32(h2), bf16_to_f32(h3));
        }
        *reinterpret_cast<float4*>(out + (size_t)c * Dp + k) = v;
    }
}

// The plain modes (copy, h + r, h * r; float32 output only) with RPW rows per wave: the kernel
// is bound by the number of resident waves times the latency of the chain row id -> row ->
// store, so a wave that keeps RPW chains in flight moves RPW times the rows in the same time.
template <int RPW>
__global__ __launch_bounds__(256) void k_gather_operands_multi(RowSource ent, const float* __restrict__ rel,
                                                               const uint32_t* __restrict__ crel, int rel_mode,
                                                               int n_head, int n_rows, int Dp,
                                                               float* __restrict__ out, TailCols tc) {
    const int lane = threadIdx.x & 63;
    const int c0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW;
    if (c0 >= n_rows) return;
    // the row numbers are asked for together with the block's tail count (rows past it are
    // never used, but their slots hold valid numbers): one round trip instead of two in front
    // of the rows themselves
    uint32_t key[RPW], rkey[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int c = min(c0 + r, n_rows - 1);  // a row past the end repeats the last one
        key[r] = ent.index ? ent.index[c] : (uint32_t)c;
        rkey[r] = (c < n_head && rel_mode) ? crel[c] : 0u;
    }
    // (limits are multiples of RPW: the rows of a wave are live or not together)
    const bool live = tc.live(c0 - n_head);
#pragma unroll
    for (int r = 0; r < RPW; ++r) asm volatile("" : "+v"(key[r]), "+v"(rkey[r]));
    if (!live) return;
    const char* row[RPW];
    const float* rrow[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int c = min(c0 + r, n_rows - 1);
        row[r] = ent.base + (int64_t)key[r] * ent.pitch;
        rrow[r] = (c < n_head && rel_mode) ? rel + (size_t)rkey[r] * Dp : nullptr;
    }
    for (int k = lane * 4; k < Dp; k += 256) {
        float4 v[RPW], q[RPW];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {  // all loads first
            v[r] = load4(row[r], k, ent);
            q[r] = rrow[r] ? *reinterpret_cast<const float4*>(rrow[r] + k) : make_float4(0, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            if (rrow[r]) v[r] = rel_mode == 1 ? f4add(v[r], q[r]) : f4mul(v[r], q[r]);
            v[r].x += 0.f; v[r].y += 0.f; v[r].z += 0.f; v[r].w += 0.f;  // -0 -> +0, as above
        }
#pragma unroll
        for (int r = 0; r < RPW; ++r)
            if (c0 + r < n_rows) *reinterpret_cast<float4*>(out + (size_t)(c0 + r) * Dp + k) = v[r];
    }
}

// rows per wave of the plain gather: 2 measured best (10.6 -> 9.2 us on the 1M-row workload,
// 22.7 -> 20.8 us on the 22.8M-row one; 4 is slower than 1)
constexpr int kGatherRowsPerWave = 2;
void launch_gather_operands(const RowSource& ent, const float* rel, const uint32_t* crel, int rel_mode,
                            int half, int n_head, int n_rows, int Dp, float* out, uint16_t* out16,
                            hipStream_t stream, const TailCols* tail_cols) {
    TailCols tc = {};
    if (tail_cols) tc = *tail_cols;
    const bool pairs_ok = !tc.tcount || (n_head % kGatherRowsPerWave == 0 && tc.T % kGatherRowsPerWave == 0 &&
                                         tc.tpad % kGatherRowsPerWave == 0);
    if (rel_mode >= 3)
        hipLaunchKernelGGL(k_gather_operands<true>, dim3((n_rows + 3) / 4), dim3(256), 0, stream, ent, rel, crel,
                           rel_mode, half, n_head, n_rows, Dp, out, out16, tc);
    else if (!out16 && n_rows >= 8192 && pairs_ok)
        hipLaunchKernelGGL(k_gather_operands_multi<kGatherRowsPerWave>,
                           dim3((n_rows + 4 * kGatherRowsPerWave - 1) / (4 * kGatherRowsPerWave)),
                           dim3(256), 0, stream, ent, rel, crel, rel_mode, n_head, n_rows, Dp, out, tc);
    else
        hipLaunchKernelGGL(k_gather_operands<false>, dim3((n_rows + 3) / 4), dim3(256), 0, stream, ent, rel, crel,
                           rel_mode, half, n_head, n_rows, Dp, out, out16, tc);
}

// --------------------------------------------------------------------------
// scoring: forward

// logSigmoid and its derivative exactly as src/pag/pag.cpp:894-903
DEVINL float log_sigmoid(float z) { return z > -11.f ? -log1pf(expf(-z)) : z; }
DEVINL float log_sigmoid_grad(float z) { return 1.f / (1.f + expf(fminf(z, 11.f))); }

// The same two functions from ONE hardware exponential (the scoring epilogues
// evaluate them once per score): with u = exp(-|z|) in (0, 1],
//   z >= 0:        logsig = -log1p(u),     dlogsig = u' / (1 + u'),  u' = max(u, e^-11)  (the +11 clamp;
//                  u / (1 + u) grows with u, so the clamp can move to the quotient)
//   -11 < z < 0:   logsig = z - log1p(u),  dlogsig = 1 / (1 + u)
//   z <= -11:      logsig = z              (the reference drops the log1p term there)
// log1p(u) = log(w) - ((w - 1) - u) / w with w = 1 + u keeps the low bits of u.
DEVINL void log_sigmoid_both(float z, float& value, float& grad) {
    // single hardware instructions: exp2, rcp and log2 (about 1 ulp each; w is in [1, 2], so
    // none of the range fix-ups of the library forms is needed)
    const float u = __builtin_amdgcn_exp2f(-1.44269504089f * fabsf(z));
    const float w = 1.f + u;
    const float rw = __builtin_amdgcn_rcpf(w);
    const float l1p = 0.69314718056f * __builtin_amdgcn_logf(w) - ((w - 1.f) - u) * rw;
    // straight-line selects (lanes of a wave mix both signs of z):
    //   value = min(z, 0) - log1p(u), without the log1p term for z <= -11
    //   grad  = u / (1 + u) clamped below at its value for u = e^-11 (z >= 0), 1 / (1 + u) (z < 0)
    value = fminf(z, 0.f) - (z > -11.f ? l1p : 0.f);
    const float g_pos = fmaxf(u * rw, 1.670142184e-5f);  // e^-11 / (1 + e^-11)
    grad = z >= 0.f ? g_pos : rw;
}

// The same for both signs of one score: exp(-|z|) serves z = s and z = -s alike.
DEVINL void log_sigmoid_pair(float s, float& v_pos, float& g_pos, float& v_neg, float& g_neg) {
    const float u = __builtin_amdgcn_exp2f(-1.44269504089f * fabsf(s));
    const float w = 1.f + u;
    const float rw = __builtin_amdgcn_rcpf(w);
    const float l1p = 0.69314718056f * __builtin_amdgcn_logf(w) - ((w - 1.f) - u) * rw;
    const float g_big = fmaxf(u * rw, 1.670142184e-5f);  // e^-11 / (1 + e^-11)
    v_pos = fminf(s, 0.f) - (s > -11.f ? l1p : 0.f);
    v_neg = fminf(-s, 0.f) - (s < 11.f ? l1p : 0.f);
    g_pos = s >= 0.f ? g_big : rw;
    g_neg = s <= 0.f ? g_big : rw;
}

// The logsigmoid loss of one score column that stands for `mult` tail positions, one of them the
// positive's label if `pos` (src/poplar_kge.cpp:615-636 summed over the positions that share the
// row): returns the loss term (before the normalisation) and sets d loss / d score (times grad_scale).
DEVINL float logsigmoid_column(float score, bool pos, float mult, float w_pos, float w_neg, float grad_scale,
                               float& dscore) {
    float v_pos, g_pos, v_neg, g_neg;
    log_sigmoid_pair(score, v_pos, g_pos, v_neg, g_neg);
    const float wp = pos ? w_pos : 0.f, wn = (mult - (pos ? 1.f : 0.f)) * w_neg;
    dscore = (wn * g_neg - wp * g_pos) * grad_scale;
    return -(wp * v_pos + wn * v_neg);
}

struct FwdParams {
    ScoreShape sh;
    RowSource ent_a, ent_b;
    const float* rel;
    const uint32_t* crel;
    const uint32_t* clabel;
    float* coef;
    float* dist;
    float* loss_part;
    int a_rel_mode;   // how the a-operand combines with its relation row
    int out_mode;     // 0 fused logsigmoid -> coefficient; 1 raw score (+dist); 2 raw distance
    int a_c0, b_c0;   // contribution index of block 0's first a / b row
    uint32_t* nearflag;  // [S, ceil(B/32), ceil(T/32)] or null: 32x32 sub-blocks holding near-identical pairs
};

constexpr int BK = 32;         // embedding columns staged per iteration

// ALIGNED: whole tiles and slabs of dense float32 operands with the relation already applied:
// the staging loads carry no bounds checks, and the next slab's are in flight while the current
// slab is worked on (86 -> 84 us on the 22.8M-row L1 workload: the other workgroups of a CU hide
// most of that latency already).
template <int DIST, int OM, bool ALIGNED = false>  // OM: FwdParams::out_mode, fixed at compile time
__global__ __launch_bounds__(256) void k_score_fwd(FwdParams p) {
    __shared__ __attribute__((aligned(16))) float As[BK][LDP];
    __shared__ __attribute__((aligned(16))) float Bs[BK][LDP];
    __shared__ float red[4];
    __shared__ uint32_t label_s[kScoreTile];
    const ScoreShape& sh = p.sh;
    const TileId tile = xcd_tile((sh.T + kScoreTile - 1) / kScoreTile, (sh.B + kScoreTile - 1) / kScoreTile, sh.S);
    const int d = tile.z, m0 = tile.y * kScoreTile, n0 = tile.x * kScoreTile;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int B = sh.B, T = sh.T, Dp = sh.Dp;
    if (n0 >= tail_limit(sh.tcount, d, T, sh.tpad)) {  // merged tails: the block has no such column
        if (OM == 0 && tid == 0) p.loss_part[(size_t)d * (tile.gx * tile.gy) + tile.y * tile.gx + tile.x] = 0.f;
        return;
    }
    if (OM == 0 && tid < kScoreTile) label_s[tid] = m0 + tid < B ? p.clabel[d * B + m0 + tid] : 0u;
    float mult[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + tx * 4 + j;
        mult[j] = (OM == 0 && sh.tmult && n < T) ? sh.tmult[(size_t)d * T + n] : 1.f;
    }

    // staging assignment: row lr of each operand, float4 columns k4 and k4 + 16.  Sixteen
    // consecutive rows per wave and four column groups: a store instruction's 64 lanes fall on
    // every LDS bank exactly twice (with eight column groups per row they met four to a bank).
    static_assert(BK == 32 && kScoreTile == 64, "the staging assignment covers 64 rows x 32 columns");
    const int lr = tid >> 2, k4 = (tid & 3) * 4;
    const int sm = m0 + lr, sn = n0 + lr;
    const char* arow = sm < B ? row_ptr(p.ent_a, p.a_c0 + d * B + sm) : nullptr;
    const float* rrow = (sm < B && p.a_rel_mode) ? p.rel + (size_t)p.crel[d * B + sm] * Dp : nullptr;
    const char* brow = sn < T ? row_ptr(p.ent_b, p.b_c0 + d * T + sn) : nullptr;

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    float4 ra[2], rb[2];
    auto prefetch = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ra[h] = *reinterpret_cast<const float4*>(arow + (size_t)(k0 + 16 * h + k4) * 4);
            rb[h] = *reinterpret_cast<const float4*>(brow + (size_t)(k0 + 16 * h + k4) * 4);
        }
    };
    if (ALIGNED) prefetch(0);
    for (int k0 = 0; k0 < Dp; k0 += BK) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int kc = 16 * h + k4, k = k0 + kc;
            float4 a = make_float4(0, 0, 0, 0), b = a;
            if (ALIGNED) {
                a = ra[h]; b = rb[h];
            } else if (k < Dp) {
                if (arow) a = combine_rel(load4(arow, k, p.ent_a), rrow, k, p.a_rel_mode);
                if (brow) b = load4(brow, k, p.ent_b);
            }
            As[kc + 0][lr] = a.x; As[kc + 1][lr] = a.y; As[kc + 2][lr] = a.z; As[kc + 3][lr] = a.w;
            Bs[kc + 0][lr] = b.x; Bs[kc + 1][lr] = b.y; Bs[kc + 2][lr] = b.z; Bs[kc + 3][lr] = b.w;
        }
        __syncthreads();
        // branch-free: past the end the last slab is loaded again
        if (ALIGNED) prefetch(min(k0 + BK, Dp - BK));
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            const float4 a4 = *reinterpret_cast<const float4*>(&As[kk][ty * 4]);
            const float4 b4 = *reinterpret_cast<const float4*>(&Bs[kk][tx * 4]);
            const float av[4] = {a4.x, a4.y, a4.z, a4.w};
            const float bv[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (DIST == DIST_L1) {
                        acc[i][j] += fabsf(av[i] - bv[j]);
                    } else if (DIST == DIST_L2) {
                        const float t = av[i] - bv[j];
                        acc[i][j] = fmaf(t, t, acc[i][j]);
                    } else {
                        acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
                    }
                }
        }
        __syncthreads();
    }

    // epilogue
    const float Tn = (float)T;
    // kept in scalar registers (see the matrix-core kernel's epilogue)
    const float w_pos = uniform_f32(0.5f * Tn), w_neg = uniform_f32((0.5f * Tn) / (float)(T - 1));
    const float inv_norm = uniform_f32(1.f / ((float)sh.S * (float)B * Tn));
    const float grad_scale = uniform_f32(inv_norm * sh.loss_scale);
    float loss_acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= B) continue;
        const uint32_t label = OM == 0 ? label_s[ty * 4 + i] : 0u;
        float outv[4], distv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            const float dist = DIST == DIST_L2 ? sqrtf(acc[i][j]) : acc[i][j];
            distv[j] = dist;
            if (OM == 2) { outv[j] = dist; continue; }
            const float score = score_is_distance_value(sh.score_fn) ? dist : sh.gamma - dist;
            if (OM == 1) { outv[j] = score; continue; }
            float ds;  // d loss / d score, times the loss scale
            const float term = logsigmoid_column(score, (uint32_t)n == label, mult[j], w_pos, w_neg, grad_scale, ds);
            if (n < T) loss_acc += term;
            float c = score_is_distance_value(sh.score_fn) ? ds : -ds;  // score = gamma - dist
            if (DIST == DIST_L2) c = dist != 0.f ? c * __builtin_amdgcn_rcpf(dist) : 0.f;
            outv[j] = c;
        }
        const int n = n0 + tx * 4;
        float* crow = p.coef + ((size_t)d * B + m) * T;
        float* drow = (OM == 1 && DIST == DIST_L2 && p.dist) ? p.dist + ((size_t)d * B + m) * T : nullptr;
        if (n + 3 < T && (T & 3) == 0) {
            *reinterpret_cast<float4*>(crow + n) = make_float4(outv[0], outv[1], outv[2], outv[3]);
            if (drow) *reinterpret_cast<float4*>(drow + n) = make_float4(distv[0], distv[1], distv[2], distv[3]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (n + j < T) {
                    crow[n + j] = outv[j];
                    if (drow) drow[n + j] = distv[j];
                }
        }
    }
    if (OM == 0) {
        loss_acc = wave_sum(loss_acc);
        if ((tid & 63) == 0) red[tid >> 6] = loss_acc;
        __syncthreads();
        if (tid == 0) {
            const int n_part = tile.gx * tile.gy;
            p.loss_part[(size_t)d * n_part + tile.y * tile.gx + tile.x] =
                (red[0] + red[1] + red[2] + red[3]) * inv_norm;
        }
    }
}

// --------------------------------------------------------------------------
// scoring forward on the matrix cores (L2 and dot): S[m,n] = sum_k a[m,k] b[n,k]
// with v_mfma_f32_32x32x2_f32.  Workgroup tile 128 (a rows) x 64 (b rows), four
// waves as 2 x 2, each wave two 32x32 accumulators.  For L2,
// d^2 = |a|^2 + |b|^2 - 2 a.b; where that cancels (d^2 small against the norms)
// the pair is recomputed directly as sum (a-b)^2 by the whole wave, so the
// result keeps float32 accuracy and is exactly 0 for identical rows.


constexpr int FM_TM = 128, FM_TN = 64;
constexpr float kCancelRatio = 0.125f;  // recompute when d^2 < ratio * (|a|^2 + |b|^2)
// Below this ratio the backward's product form self*sum(c) - sum(c*other) would
// lose accuracy against the reference's c*(self-other); such 32x32 sub-blocks
// are flagged for the backward kernel, which handles them in the direct form.
constexpr float kNearRatio = 1.f / 4096.f;

// BKT = embedding columns staged per iteration: with 128 a whole D = 256 row
// takes two iterations, the loads of the second in flight under the first's
// matrix work (99 KB of LDS).  NW = waves per workgroup: 8 (two per SIMD, each
// one 32x32 accumulator) when a launch has so few workgroups that each CU gets
// one, so that a second wave hides the other's LDS and epilogue latencies; 4
// (each two accumulators) otherwise.
// ALIGNED: B % 128 == 0, T % 64 == 0, Dp % BKT == 0, dense float32 operands with
// the relation already applied: the staging loads carry no bounds checks (and
// so no branches that would force the prefetch to complete before the matrix
// work starts).
// OM: what the epilogue stores (FwdParams::out_mode), a template parameter so that the
// sixteen outputs of a lane form one straight-line block the scheduler can interleave
// SPLIT: the products run as six bfloat16 matrix instructions on three-piece operands
// (split4_bf16): the tiles hold the three pieces of every value, split while staging.
// PF: slabs of operand loads in flight (register sets).  A slab's loads take a round trip to the
// memory-side cache however little work the slab is, so with PF = 1 that latency is paid per slab.
template <int DIST, int BKT, bool ALIGNED, int NW, int OM, bool SPLIT = false, int PF = 1>
__global__ __launch_bounds__(NW * 64) void k_score_fwd_mfma(FwdParams p) {
    constexpr int NT = NW * 64;       // threads
    constexpr int AT = 8 / NW;        // 32-row accumulator tiles per wave (NW/2 waves cover 128 rows)
    constexpr int RP = NT / 8;        // rows staged per pass (8 threads share a row)
    constexpr int HA = FM_TM / RP, HB = FM_TN / RP;
    constexpr int NC = BKT / 32;      // float4 columns per staged row per thread
    // tiles keep the operands' own layout (row = entity row, columns contiguous):
    // staging is a float4 copy, and a lane fetches four consecutive columns of
    // its row in one 16-byte LDS read that feeds four matrix instructions.  The
    // pitch of BKT + 4 floats spreads eight consecutive rows over all banks.
    constexpr int LDT = BKT + 4;
    __shared__ __attribute__((aligned(16))) float As[SPLIT ? 1 : FM_TM][LDT];
    __shared__ __attribute__((aligned(16))) float Bs[SPLIT ? 1 : FM_TN][LDT];
    // SPLIT: two copies of [piece][row][32 columns] bfloat16; rows of 64 bytes whose four
    // 16-byte chunks are stored at position chunk ^ ((row / 4) % 4), which puts sixteen
    // consecutive rows' reads of one chunk in different banks without padding
    __shared__ __attribute__((aligned(16))) uint16_t Ap[SPLIT ? 2 : 1][SPLIT ? 3 : 1][SPLIT ? FM_TM : 1][BKT];
    __shared__ __attribute__((aligned(16))) uint16_t Bp[SPLIT ? 2 : 1][SPLIT ? 3 : 1][SPLIT ? FM_TN : 1][BKT];
    __shared__ float na_s[FM_TM], nb_s[FM_TN];
    __shared__ float red[NW];
    __shared__ uint32_t label_s[FM_TM];
    const ScoreShape& sh = p.sh;
    const TileId tile = xcd_tile((sh.T + FM_TN - 1) / FM_TN, (sh.B + FM_TM - 1) / FM_TM, sh.S);
    const int d = tile.z, m0 = tile.y * FM_TM, n0 = tile.x * FM_TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * (32 * AT), wn = (wave & 1) * 32;
    const int B = sh.B, T = sh.T, Dp = sh.Dp;
    if (n0 >= tail_limit(sh.tcount, d, T, sh.tpad)) {  // merged tails: the block has no such column
        if (OM == 0 && tid == 0) p.loss_part[(size_t)d * (tile.gx * tile.gy) + tile.y * tile.gx + tile.x] = 0.f;
        return;
    }
    if (OM == 0 && tid < FM_TM) label_s[tid] = m0 + tid < B ? p.clabel[d * B + m0 + tid] : 0u;

    const int srow = tid >> 3, k4 = (tid & 7) * 4;
    const char* arow[HA];
    const float* rrow[HA];
    const char* brow[HB];
#pragma unroll
    for (int h = 0; h < HA; ++h) {
        const int m = m0 + srow + RP * h;
        if (ALIGNED) {  // dense, un-indexed operands: plain address arithmetic
            arow[h] = p.ent_a.base + (int64_t)(p.a_c0 + d * B + m) * p.ent_a.pitch;
            rrow[h] = nullptr;
        } else {
            arow[h] = m < B ? row_ptr(p.ent_a, p.a_c0 + d * B + m) : nullptr;
            rrow[h] = (m < B && p.a_rel_mode) ? p.rel + (size_t)p.crel[d * B + m] * Dp : nullptr;
        }
    }
#pragma unroll
    for (int h = 0; h < HB; ++h) {
        const int n = n0 + srow + RP * h;
        if (ALIGNED) brow[h] = p.ent_b.base + (int64_t)(p.b_c0 + d * T + n) * p.ent_b.pitch;
        else brow[h] = n < T ? row_ptr(p.ent_b, p.b_c0 + d * T + n) : nullptr;
    }
    float na_acc[HA], nb_acc[HB];
#pragma unroll
    for (int h = 0; h < HA; ++h) na_acc[h] = 0.f;
#pragma unroll
    for (int h = 0; h < HB; ++h) nb_acc[h] = 0.f;
    floatx16 acc[AT];
#pragma unroll
    for (int t = 0; t < AT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;

    floatx4 areg[PF][HA][NC], breg[PF][HB][NC];
    auto prefetch = [&](auto set, int k0) __attribute__((always_inline)) {
        constexpr int s = decltype(set)::value;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int k = k0 + 32 * c + k4;
            if (ALIGNED) {
#pragma unroll
                for (int h = 0; h < HA; ++h) areg[s][h][c] = *reinterpret_cast<const floatx4*>(arow[h] + (size_t)k * 4);
#pragma unroll
                for (int h = 0; h < HB; ++h) breg[s][h][c] = *reinterpret_cast<const floatx4*>(brow[h] + (size_t)k * 4);
                continue;
            }
#pragma unroll
            for (int h = 0; h < HA; ++h) {
                areg[s][h][c] = floatx4{0.f, 0.f, 0.f, 0.f};
                if (arow[h] && k < Dp)
                    areg[s][h][c] = as_x4(combine_rel(load4(arow[h], k, p.ent_a), rrow[h], k, p.a_rel_mode));
            }
#pragma unroll
            for (int h = 0; h < HB; ++h) {
                breg[s][h][c] = floatx4{0.f, 0.f, 0.f, 0.f};
                if (brow[h] && k < Dp) breg[s][h][c] = as_x4(load4(brow[h], k, p.ent_b));
            }
        }
    };
    static_for<PF>([&](auto set) {
        if (ALIGNED || decltype(set)::value * BKT < Dp) prefetch(set, decltype(set)::value * BKT);
    });
    if constexpr (SPLIT) {
        static_assert(BKT == 32 && PF % 2 == 0 && ALIGNED, "the three-piece path: aligned shapes, slabs of 32");
        const int hl = lane >> 5, cl = lane & 31;
        // writes one register set (a slab) into tile copy `buf`, as pieces; `live` = 0 for the
        // slab past the end (its squares must not count)
        auto stage = [&](auto set, auto bufc, float live) __attribute__((always_inline)) {
            constexpr int s = decltype(set)::value, buf = decltype(bufc)::value;
#pragma unroll
            for (int h = 0; h < HA; ++h) {
                const int row = srow + RP * h;
                const int col = (((k4 >> 3) ^ ((row >> 2) & 3)) << 3) + (k4 & 4);
                const floatx4 a = areg[s][h][0];
                uint2 piece[3];
                split4_bf16(a, piece);
#pragma unroll
                for (int q = 0; q < 3; ++q) *reinterpret_cast<uint2*>(&Ap[buf][q][row][col]) = piece[q];
                if (DIST == DIST_L2) na_acc[h] += live * (a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w);
            }
#pragma unroll
            for (int h = 0; h < HB; ++h) {
                const int row = srow + RP * h;
                const int col = (((k4 >> 3) ^ ((row >> 2) & 3)) << 3) + (k4 & 4);
                const floatx4 b = breg[s][h][0];
                uint2 piece[3];
                split4_bf16(b, piece);
#pragma unroll
                for (int q = 0; q < 3; ++q) *reinterpret_cast<uint2*>(&Bp[buf][q][row][col]) = piece[q];
                if (DIST == DIST_L2) nb_acc[h] += live * (b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w);
            }
        };
        using I0 = std::integral_constant<int, 0>;
        stage(I0{}, I0{}, 1.f);
        prefetch(I0{}, min(PF * BKT, Dp - BKT));
        __syncthreads();
        // One barrier per slab: while the matrix cores work on one tile copy the next slab is
        // split into the other, the splitting instructions issued between the matrix
        // instructions (each of which depends on the one before it).
        for (int kb = 0; kb < Dp; kb += PF * BKT)
        static_for<PF>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            using Next = std::integral_constant<int, (s + 1) % PF>;
            using Other = std::integral_constant<int, (s + 1) & 1>;
            constexpr int buf = s & 1;
            const int k0 = kb + s * BKT;
            // the slab in tile copy `buf`: two steps of sixteen columns; a lane supplies columns
            // 8 * (lane / 32) .. + 7 of a step, of its row, for both operands
            floatx4 fa[2][AT][3], fb[2][3];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const int chunk = 2 * ks + hl;
#pragma unroll
                for (int q = 0; q < 3; ++q) {
                    const int rb = wn + cl;
                    fb[ks][q] = *reinterpret_cast<const floatx4*>(&Bp[buf][q][rb][(chunk ^ ((rb >> 2) & 3)) << 3]);
#pragma unroll
                    for (int t = 0; t < AT; ++t) {
                        const int ra = wm + 32 * t + cl;
                        fa[ks][t][q] = *reinterpret_cast<const floatx4*>(&Ap[buf][q][ra][(chunk ^ ((ra >> 2) & 3)) << 3]);
                    }
                }
            }
            stage(Next{}, Other{}, k0 + BKT < Dp ? 1.f : 0.f);
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int t = 0; t < AT; ++t) acc[t] = mfma_split6(fa[ks][t], fb[ks], acc[t]);
            // the order asked of the scheduler: the LDS reads, then one matrix instruction,
            // a share of the vector work and an LDS write, in turn
            __builtin_amdgcn_sched_group_barrier(0x100, 6 * (AT + 1), 0);
#pragma unroll
            for (int i = 0; i < 12 * AT; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, (30 * (HA + HB) + 12 * AT - 1) / (12 * AT), 0);
                if (i < 3 * (HA + HB)) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
            }
            prefetch(Next{}, min(k0 + BKT + PF * BKT, Dp - BKT));
            __syncthreads();
        });
    } else
    for (int kb = 0; kb < Dp; kb += PF * BKT)
    static_for<PF>([&](auto set) {
        constexpr int s = decltype(set)::value;
        const int k0 = kb + s * BKT;
        if (!ALIGNED && PF > 1 && k0 >= Dp) return;  // ALIGNED: Dp % (PF * BKT) == 0
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int kc = 32 * c + k4;
#pragma unroll
            for (int h = 0; h < HA; ++h) {
                const float4 a = as_f4(areg[s][h][c]);
                *reinterpret_cast<float4*>(&As[srow + RP * h][kc]) = a;
                if (DIST == DIST_L2) na_acc[h] += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
            }
#pragma unroll
            for (int h = 0; h < HB; ++h) {
                const float4 b = as_f4(breg[s][h][c]);
                *reinterpret_cast<float4*>(&Bs[srow + RP * h][kc]) = b;
                if (DIST == DIST_L2) nb_acc[h] += b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
            }
        }
        __syncthreads();
        // ALIGNED: branch-free (a branch here would merge the register set's old and new
        // contents and wait for the loads at once); past the end the last slab is loaded again
        if (ALIGNED) prefetch(set, min(k0 + PF * BKT, Dp - BKT));
        else if (k0 + PF * BKT < Dp) prefetch(set, k0 + PF * BKT);
        // Each group of four matrix instructions covers eight columns: instruction
        // x takes column 8g + x from the lower half-wave and 8g + 4 + x from the
        // upper one.  Operands are fetched one group ahead of their use.
        {
            constexpr int NG = BKT / 8;
            float4 ra[2][AT], rb[2];
            const int hl = lane >> 5, cl = lane & 31;
            rb[0] = *reinterpret_cast<const float4*>(&Bs[wn + cl][4 * hl]);
#pragma unroll
            for (int t = 0; t < AT; ++t) ra[0][t] = *reinterpret_cast<const float4*>(&As[wm + 32 * t + cl][4 * hl]);
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                if (g + 1 < NG) {
                    rb[(g + 1) & 1] = *reinterpret_cast<const float4*>(&Bs[wn + cl][8 * (g + 1) + 4 * hl]);
#pragma unroll
                    for (int t = 0; t < AT; ++t)
                        ra[(g + 1) & 1][t] =
                            *reinterpret_cast<const float4*>(&As[wm + 32 * t + cl][8 * (g + 1) + 4 * hl]);
                }
                __builtin_amdgcn_sched_barrier(0);
                const float bx[4] = {rb[g & 1].x, rb[g & 1].y, rb[g & 1].z, rb[g & 1].w};
#pragma unroll
                for (int t = 0; t < AT; ++t) {
                    const float ax[4] = {ra[g & 1][t].x, ra[g & 1][t].y, ra[g & 1][t].z, ra[g & 1][t].w};
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(ax[x], bx[x], acc[t], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    });
    if (DIST == DIST_L2) {
        // the 8 threads of a row hold partial sums of squares: combine in a fixed order
#pragma unroll
        for (int h = 0; h < HA; ++h) {
            float v = na_acc[h];
            v += __shfl_xor(v, 1, 64); v += __shfl_xor(v, 2, 64); v += __shfl_xor(v, 4, 64);
            if ((tid & 7) == 0) na_s[srow + RP * h] = v;
        }
#pragma unroll
        for (int h = 0; h < HB; ++h) {
            float v = nb_acc[h];
            v += __shfl_xor(v, 1, 64); v += __shfl_xor(v, 2, 64); v += __shfl_xor(v, 4, 64);
            if ((tid & 7) == 0) nb_s[srow + RP * h] = v;
        }
        __syncthreads();
    }

    // epilogue.  Accumulator layout of v_mfma_f32_32x32x2_f32: register r of
    // lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32.
    const float Tn = (float)T;
    // loss weights and the gradient scale, kept in scalar registers so that the compiler
    // does not re-derive them (a division each) at every output
    const float w_pos = uniform_f32(0.5f * Tn), w_neg = uniform_f32((0.5f * Tn) / (float)(T - 1));
    const float inv_norm = uniform_f32(1.f / ((float)sh.S * (float)B * Tn));
    const float grad_scale = uniform_f32(inv_norm * sh.loss_scale);
    float loss_acc = 0.f;
    const int n_loc = wn + (lane & 31), n = n0 + n_loc;
    // outputs of this block: 32-bit offsets inside the block's [B, T] matrix
    float* const coef_blk = p.coef + (size_t)d * B * T;
    float* const dist_blk = p.dist ? p.dist + (size_t)d * B * T : nullptr;
    const float nb = DIST == DIST_L2 ? nb_s[n_loc] : 0.f;
    const float mult = (OM == 0 && sh.tmult && n < T) ? sh.tmult[(size_t)d * T + n] : 1.f;
#pragma unroll
    for (int t = 0; t < AT; ++t) {
        // phase 1 (straight-line): squared distances and which of them cancelled
        float val[16];
        uint32_t cancel = 0u, near = 0u;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m_loc = wm + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            const bool live = ALIGNED || (m0 + m_loc < B && n < T);
            val[r] = acc[t][r];
            if (DIST == DIST_L2) {
                const float na = na_s[m_loc];
                val[r] = na + nb - 2.f * acc[t][r];
                if (live && val[r] < kCancelRatio * (na + nb)) cancel |= 1u << r;
                if (live && val[r] < kNearRatio * (na + nb)) near |= 1u << r;
            }
        }
        // phase 2 (rare): the wave recomputes the cancelled pairs directly
        if (DIST == DIST_L2 && __ballot(cancel != 0u)) {
            near = 0u;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m_loc = wm + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                const int m = m0 + m_loc;
                uint64_t todo = __ballot((cancel >> r) & 1u);
                while (todo) {
                    const int src = __ffsll((long long)todo) - 1;
                    todo &= todo - 1;
                    const int fm = __shfl(m, src, 64), fn = __shfl(n, src, 64);
                    const char* ar = row_ptr(p.ent_a, p.a_c0 + d * B + fm);
                    const float* rr = p.a_rel_mode ? p.rel + (size_t)p.crel[d * B + fm] * Dp : nullptr;
                    const char* br = row_ptr(p.ent_b, p.b_c0 + d * T + fn);
                    float part = 0.f;
                    for (int k = lane * 4; k < Dp; k += 256) {
                        const float4 a = combine_rel(load4(ar, k, p.ent_a), rr, k, p.a_rel_mode);
                        const float4 b = load4(br, k, p.ent_b);
                        const float dx = a.x - b.x, dy = a.y - b.y, dz = a.z - b.z, dw = a.w - b.w;
                        part += dx * dx + dy * dy + dz * dz + dw * dw;
                    }
                    part = wave_sum(part);
                    if (lane == src) val[r] = part;
                }
                const bool live = ALIGNED || (m < B && n < T);
                if (live && val[r] < kNearRatio * (na_s[m_loc] + nb)) near |= 1u << r;
            }
        }
        // phase 3 (straight-line): distance, score, loss, backward coefficient
        uint32_t label_r[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
            label_r[r] = OM == 0 ? label_s[wm + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)] : 0u;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m_loc = wm + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            const int m = m0 + m_loc;
            const bool live = ALIGNED || (m < B && n < T);
            const float dist = DIST == DIST_L2 ? __builtin_amdgcn_sqrtf(fmaxf(val[r], 0.f)) : val[r];
            float outv;
            if (OM == 2) {
                outv = dist;
            } else {
                const float score = score_is_distance_value(sh.score_fn) ? dist : sh.gamma - dist;
                if (OM == 1) {
                    outv = score;
                    if (live && DIST == DIST_L2 && dist_blk) dist_blk[m * T + n] = dist;
                } else {
                    float ds;
                    const float term = logsigmoid_column(score, (uint32_t)n == label_r[r], mult, w_pos, w_neg, grad_scale, ds);
                    if (live) loss_acc += term;
                    outv = score_is_distance_value(sh.score_fn) ? ds : -ds;
                    if (DIST == DIST_L2) outv = dist != 0.f ? outv * __builtin_amdgcn_rcpf(dist) : 0.f;
                }
            }
            if (live) coef_blk[m * T + n] = outv;
        }
        if (DIST == DIST_L2 && p.nearflag) {
            // this wave owns the whole 32x32 sub-block: a plain store, no atomics
            const bool any = __ballot(near != 0u) != 0;
            const int mt = (m0 + wm + 32 * t) >> 5, nt = (n0 + wn) >> 5;
            const int MT = (B + 31) >> 5, NTL = (T + 31) >> 5;
            if (lane == 0 && mt < MT && nt < NTL) p.nearflag[((size_t)d * MT + mt) * NTL + nt] = any ? 1u : 0u;
        }
    }
    if (OM == 0) {
        loss_acc = wave_sum(loss_acc);
        if (lane == 0) red[wave] = loss_acc;
        __syncthreads();
        if (tid == 0) {
            const int n_part = tile.gx * tile.gy;
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) tot += red[w];
            p.loss_part[(size_t)d * n_part + tile.y * tile.gx + tile.x] = tot * inv_norm;
        }
    }
}

static bool fwd_uses_mfma(const FwdParams& p) {
    return p.sh.use_mfma && p.sh.dist_fn != DIST_L1 && p.ent_a.vec && p.ent_b.vec && (p.sh.Dp & 3) == 0;
}

int score_fwd_parts(const ScoreShape& sh) {
    const bool mfma = sh.use_mfma && !(sh.score_fn != SCORE_DISTMULT && sh.dist_fn == DIST_L1);
    const int tm = mfma ? FM_TM : kScoreTile, tn = mfma ? FM_TN : kScoreTile;
    return ((sh.T + tn - 1) / tn) * ((sh.B + tm - 1) / tm);
}

static void launch_fwd(const FwdParams& p, hipStream_t stream) {
    if (fwd_uses_mfma(p)) {
        const dim3 grid = tile_grid((p.sh.T + FM_TN - 1) / FM_TN, (p.sh.B + FM_TM - 1) / FM_TM, p.sh.S);
        const bool f32 = p.ent_a.etype == ET_F32 && p.ent_b.etype == ET_F32;
        const bool aligned = f32 && p.a_rel_mode == 0 && !p.ent_a.index && !p.ent_b.index &&
                             p.sh.B % FM_TM == 0 && p.sh.T % FM_TN == 0;
#define KGE_FWD_OM(D_, OM_)                                                                                  \
    do {                                                                                                     \
        if (aligned && p.sh.Dp % 64 == 0 && p.sh.use_mfma == 2) {                                            \
            hipLaunchKernelGGL((k_score_fwd_mfma<D_, 32, true, 8, OM_, true, 2>), grid, dim3(512), 0, stream, p); \
        }                                                                                                    \
        else if (aligned && p.sh.Dp % 32 == 0) /* eight waves: two per SIMD hide each other's latencies */ \
            hipLaunchKernelGGL((k_score_fwd_mfma<D_, 32, true, 8, OM_>), grid, dim3(512), 0, stream, p);      \
        else hipLaunchKernelGGL((k_score_fwd_mfma<D_, 32, false, 4, OM_>), grid, dim3(256), 0, stream, p);    \
    } while (0)
#define KGE_FWD(D_)                                                                                          \
    do {                                                                                                     \
        if (p.out_mode == 0) KGE_FWD_OM(D_, 0);                                                              \
        else if (p.out_mode == 1) KGE_FWD_OM(D_, 1);                                                         \
        else KGE_FWD_OM(D_, 2);                                                                              \
    } while (0)
        if (p.sh.dist_fn == DIST_L2) KGE_FWD(DIST_L2); else KGE_FWD(DIST_DOT);
#undef KGE_FWD_OM
#undef KGE_FWD
        return;
    }
    const dim3 grid = tile_grid((p.sh.T + kScoreTile - 1) / kScoreTile, (p.sh.B + kScoreTile - 1) / kScoreTile, p.sh.S);
    const bool valu_aligned = p.ent_a.etype == ET_F32 && p.ent_b.etype == ET_F32 && p.ent_a.vec && p.ent_b.vec &&
                              !p.ent_a.index && !p.ent_b.index && p.a_rel_mode == 0 &&
                              p.sh.B % kScoreTile == 0 && p.sh.T % kScoreTile == 0 && p.sh.Dp % BK == 0;
#define KGE_FWD_VALU(D_)                                                                                     \
    do {                                                                                                     \
        if (p.out_mode == 0 && valu_aligned) hipLaunchKernelGGL((k_score_fwd<D_, 0, true>), grid, dim3(256), 0, stream, p); \
        else if (p.out_mode == 0) hipLaunchKernelGGL((k_score_fwd<D_, 0>), grid, dim3(256), 0, stream, p);    \
        else if (p.out_mode == 1) hipLaunchKernelGGL((k_score_fwd<D_, 1>), grid, dim3(256), 0, stream, p);    \
        else hipLaunchKernelGGL((k_score_fwd<D_, 2>), grid, dim3(256), 0, stream, p);                         \
    } while (0)
    if (p.sh.dist_fn == DIST_L1) KGE_FWD_VALU(DIST_L1);
    else if (p.sh.dist_fn == DIST_L2) KGE_FWD_VALU(DIST_L2);
    else KGE_FWD_VALU(DIST_DOT);
#undef KGE_FWD_VALU
}

void launch_score_fwd(const ScoreShape& sh, const RowSource& ent, const float* rel,
                      const uint32_t* crel, const uint32_t* clabel, float* coef, float* dist,
                      uint32_t* nearflag, float* loss_part, bool fused_loss, hipStream_t stream) {
    FwdParams p;
    p.nearflag = nearflag;
    p.sh = sh;
    if (sh.score_fn == SCORE_DISTMULT) p.sh.dist_fn = DIST_DOT;
    p.ent_a = ent; p.ent_b = ent; p.rel = rel; p.crel = crel; p.clabel = clabel;
    p.coef = coef; p.dist = dist; p.loss_part = loss_part;
    p.a_rel_mode = sh.operands_dense ? 0 : (sh.score_fn == SCORE_DISTMULT ? 2 : 1);
    p.out_mode = fused_loss ? 0 : 1;
    p.a_c0 = 0; p.b_c0 = sh.S * sh.B;
    launch_fwd(p, stream);
}

// Raw scores of prepared rows `a` (rows 0 .. S*B) against rows `b` (rows 0 .. S*T) of another
// source, e.g. consecutive rows of the table itself: no copy of the b side is made.
void launch_score_fwd_rows(const ScoreShape& sh, const RowSource& a, const RowSource& b, float* scores,
                           hipStream_t stream) {
    FwdParams p;
    p.nearflag = nullptr;
    p.sh = sh;
    if (sh.score_fn == SCORE_DISTMULT) p.sh.dist_fn = DIST_DOT;
    p.ent_a = a; p.ent_b = b; p.rel = nullptr; p.crel = nullptr; p.clabel = nullptr;
    p.coef = scores; p.dist = nullptr; p.loss_part = nullptr;
    p.a_rel_mode = 0; p.out_mode = 1;
    p.a_c0 = 0; p.b_c0 = 0;
    launch_fwd(p, stream);
}


// --------------------------------------------------------------------------
// bfloat16 matrix-core products (execution.scoring_dtype = "bfloat16"):
//   C[z][m, n] = sum_k A[z][m, k] * Bt[z][n, k],  bfloat16 in, float32 out,
// with v_mfma_f32_32x32x16_bf16 (lane l supplies row l%32, columns
// 8*(l/32) .. +7 of the 16-column step, for both operands).  Workgroup tile
// TM x TN (128 or 64 each), four waves as 2 x 2, each (TM/64) x (TN/64)
// accumulators of 32 x 32; K slabs of 64 staged through LDS with 16-byte copies, the
// next slab in registers while the current one is multiplied.  LDS rows are padded to
// 72 elements (144 B) so that eight consecutive rows' 16-byte reads fall in different
// banks.  The launcher takes the largest tile that still gives the chip enough
// workgroups: the step's products are small, and a launch with fewer workgroups than
// CUs is bound by the latency of its slabs, not by the matrix cores.
// Shapes: M % 64 == 0, N % 64 == 0, K % 64 == 0, rows 16-byte aligned.
constexpr int GB_K = 64, GB_LD = GB_K + 8;

// AK / BK: the operand lies with the contraction index outermost (A[k][m] / B[k][n], pitch lda /
// ldb between k rows), as the other operand of a product whose result is needed transposed
// does: a thread then fetches eight k of a pair of adjacent rows with eight 4-byte loads
// (consecutive lanes on consecutive pairs) and regroups them into the two rows' 16-byte pieces
// with byte permutes, so the LDS tiles and the matrix loop are the same in every form.
// BK = 2: such a B operand in float32 (8-byte loads of a pair's two values), rounded to bfloat16
// (to nearest even) while it is regrouped.
template <bool AK, int BK, int TM, int TN>
__global__ __launch_bounds__(256) void k_gemm_nt_bf16(GemmNT g) {
    static_assert((TM == 128 || TM == 64) && (TN == 128 || TN == 64), "tile sizes");
    constexpr int NI = TM / 64, NJ = TN / 64;  // 32 x 32 accumulators per wave
    __shared__ __attribute__((aligned(16))) uint16_t As[TM][GB_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[TN][GB_LD];
    // z = batch * ksplit + split: with ksplit > 1 every split multiplies its own K / ksplit
    // columns into its own partial output [batch][split][M, N]
    const TileId tile = xcd_tile(g.N / TN, g.M / TM, g.batches * g.ksplit);
    const int zb = tile.z / g.ksplit, zs = tile.z - zb * g.ksplit;
    const int m0 = tile.y * TM, n0 = tile.x * TN;
    const int lim = zb * g.limit_stride;
    if (g.m_limit && (uint32_t)m0 >= g.m_limit[lim]) return;
    if (g.n_limit && (uint32_t)n0 >= g.n_limit[lim]) return;
    int K = g.K / g.ksplit;
    if (g.k_limit) {  // this split's share of the live columns, in whole slabs
        const int live = (int)((g.k_limit[lim] + GB_K - 1) / GB_K) * GB_K;
        K = max(0, min(K, live - zs * K));
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * (TM / 2), wn = (wave & 1) * (TN / 2);
    const int hl = lane >> 5, cl = lane & 31;
    const size_t ks0 = (size_t)zs * (g.K / g.ksplit);  // this split's first contraction index
    const uint16_t* A = g.A + (size_t)zb * g.a_batch + (AK ? ks0 * g.lda + m0 : (size_t)m0 * g.lda + ks0);
    const uint16_t* Bt = g.Bt + (BK == 2 ? 2 : 1) * ((size_t)zb * g.b_batch + (BK ? ks0 * g.ldb + n0 : (size_t)n0 * g.ldb + ks0));

    floatx16 acc[NI][NJ];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // staging: a T x 64 operand tile = 8 T 16-byte pieces, T / 32 per thread.
    // Row-major operand: piece h = row (tid + 256 h) / 8, columns 8 ((tid + 256 h) % 8) .. + 7.
    // k-outermost operand: T / 2 pairs of adjacent rows times eight 8-column groups = T / 64
    // tasks per thread; a task's lanes take consecutive pairs (all 64 of one group for T = 128,
    // 32 of each of two groups for T = 64), registers 2 t, 2 t + 1 hold its eight loaded words.
    floatx4 areg[TM / 32], breg[BK == 2 ? TN / 16 : TN / 32];
    auto task_pair = [&](int T) { return T == 128 ? lane : (lane & 31); };
    auto task_group = [&](int T, int t) { return T == 128 ? wave + 4 * t : 2 * wave + (lane >> 5); };
    auto load_kmajor = [&](auto tc, const uint16_t* X, int64_t ld, int k0, floatx4* reg) __attribute__((always_inline)) {
        constexpr int T = decltype(tc)::value;
#pragma unroll
        for (int t = 0; t < T / 64; ++t) {
            const uint16_t* src = X + (size_t)(k0 + 8 * task_group(T, t)) * ld + 2 * task_pair(T);
#pragma unroll
            for (int x = 0; x < 8; ++x)
                reg[2 * t + (x >> 2)][x & 3] = __uint_as_float(*reinterpret_cast<const uint32_t*>(src + (size_t)x * ld));
        }
    };
    auto store_kmajor = [&](auto tc, uint16_t (*Xs)[GB_LD], const floatx4* reg) __attribute__((always_inline)) {
        constexpr int T = decltype(tc)::value;
#pragma unroll
        for (int t = 0; t < T / 64; ++t) {
            uint32_t w[8];
#pragma unroll
            for (int x = 0; x < 8; ++x) w[x] = __float_as_uint(reg[2 * t + (x >> 2)][x & 3]);
            uint4 even, odd;  // the lower halves (row 2 pair) and the upper halves (row 2 pair + 1)
            even.x = __builtin_amdgcn_perm(w[1], w[0], 0x05040100u); odd.x = __builtin_amdgcn_perm(w[1], w[0], 0x07060302u);
            even.y = __builtin_amdgcn_perm(w[3], w[2], 0x05040100u); odd.y = __builtin_amdgcn_perm(w[3], w[2], 0x07060302u);
            even.z = __builtin_amdgcn_perm(w[5], w[4], 0x05040100u); odd.z = __builtin_amdgcn_perm(w[5], w[4], 0x07060302u);
            even.w = __builtin_amdgcn_perm(w[7], w[6], 0x05040100u); odd.w = __builtin_amdgcn_perm(w[7], w[6], 0x07060302u);
            const int col = 8 * task_group(T, t), row = 2 * task_pair(T);
            *reinterpret_cast<uint4*>(&Xs[row][col]) = even;
            *reinterpret_cast<uint4*>(&Xs[row + 1][col]) = odd;
        }
    };
    // float32 source: a task's eight rows of two floats in registers 4 t .. 4 t + 3
    auto load_kmajor_f32 = [&](auto tc, const float* X, int64_t ld, int k0, floatx4* reg) __attribute__((always_inline)) {
        constexpr int T = decltype(tc)::value;
#pragma unroll
        for (int t = 0; t < T / 64; ++t) {
            const float* src = X + (size_t)(k0 + 8 * task_group(T, t)) * ld + 2 * task_pair(T);
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                const float2 v = *reinterpret_cast<const float2*>(src + (size_t)x * ld);
                reg[4 * t + (x >> 1)][2 * (x & 1)] = v.x;
                reg[4 * t + (x >> 1)][2 * (x & 1) + 1] = v.y;
            }
        }
    };
    auto store_kmajor_f32 = [&](auto tc, uint16_t (*Xs)[GB_LD], const floatx4* reg) __attribute__((always_inline)) {
        constexpr int T = decltype(tc)::value;
#pragma unroll
        for (int t = 0; t < T / 64; ++t) {
            uint32_t even[4], odd[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {  // rows 2 q, 2 q + 1 of the eight: (x, y) (x, y)
                even[q] = pack_bf16(reg[4 * t + q][0], reg[4 * t + q][2]);
                odd[q] = pack_bf16(reg[4 * t + q][1], reg[4 * t + q][3]);
            }
            const int col = 8 * task_group(T, t), row = 2 * task_pair(T);
            *reinterpret_cast<uint4*>(&Xs[row][col]) = make_uint4(even[0], even[1], even[2], even[3]);
            *reinterpret_cast<uint4*>(&Xs[row + 1][col]) = make_uint4(odd[0], odd[1], odd[2], odd[3]);
        }
    };
    using TMc = std::integral_constant<int, TM>;
    using TNc = std::integral_constant<int, TN>;
    auto prefetch = [&](int k0) __attribute__((always_inline)) {
        if (AK) load_kmajor(TMc{}, A, g.lda, k0, areg);
        if (BK == 1) load_kmajor(TNc{}, Bt, g.ldb, k0, breg);
        if (BK == 2) load_kmajor_f32(TNc{}, reinterpret_cast<const float*>(Bt), g.ldb, k0, breg);
        if (!AK) {
#pragma unroll
            for (int h = 0; h < TM / 32; ++h) {
                const int idx = tid + 256 * h, row = idx >> 3, col = (idx & 7) * 8;
                areg[h] = *reinterpret_cast<const floatx4*>(A + (size_t)row * g.lda + k0 + col);
            }
        }
        if (!BK) {
#pragma unroll
            for (int h = 0; h < TN / 32; ++h) {
                const int idx = tid + 256 * h, row = idx >> 3, col = (idx & 7) * 8;
                breg[h] = *reinterpret_cast<const floatx4*>(Bt + (size_t)row * g.ldb + k0 + col);
            }
        }
    };
    if (K > 0) prefetch(0);
    for (int k0 = 0; k0 < K; k0 += GB_K) {
        if (AK) store_kmajor(TMc{}, As, areg);
        if (BK == 1) store_kmajor(TNc{}, Bs, breg);
        if (BK == 2) store_kmajor_f32(TNc{}, Bs, breg);
        if (!AK) {
#pragma unroll
            for (int h = 0; h < TM / 32; ++h) {
                const int idx = tid + 256 * h, row = idx >> 3, col = (idx & 7) * 8;
                *reinterpret_cast<floatx4*>(&As[row][col]) = areg[h];
            }
        }
        if (!BK) {
#pragma unroll
            for (int h = 0; h < TN / 32; ++h) {
                const int idx = tid + 256 * h, row = idx >> 3, col = (idx & 7) * 8;
                *reinterpret_cast<floatx4*>(&Bs[row][col]) = breg[h];
            }
        }
        __syncthreads();
        if (k0 + GB_K < K) prefetch(k0 + GB_K);
        floatx4 fa[2][NI], fb[2][NJ];
        auto fetch = [&](int buf, int ks) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < NI; ++i) fa[buf][i] = *reinterpret_cast<const floatx4*>(&As[wm + 32 * i + cl][16 * ks + 8 * hl]);
#pragma unroll
            for (int j = 0; j < NJ; ++j) fb[buf][j] = *reinterpret_cast<const floatx4*>(&Bs[wn + 32 * j + cl][16 * ks + 8 * hl]);
        };
        fetch(0, 0);
#pragma unroll
        for (int ks = 0; ks < GB_K / 16; ++ks) {
            if (ks + 1 < GB_K / 16) fetch((ks + 1) & 1, ks + 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                        __builtin_bit_cast(bf16x8, fa[ks & 1][i]), __builtin_bit_cast(bf16x8, fb[ks & 1][j]),
                        acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    }
    // accumulator register r of lane l: row 8*(r/4) + 4*(l/32) + r%4, column l%32
    float* C = g.ksplit > 1 ? g.part + ((size_t)zb * g.ksplit + zs) * ((size_t)g.M * g.ldc)
                            : g.C + (size_t)zb * g.c_batch;
    float* __restrict__ const Cr = C;
    if (g.add_base) {
        // the added rows: all row ids first, then all values, then the stores, so that the
        // loads of one 32-row half are in flight together (in the natural order every row's
        // value waits for its id, 32 round trips one after the other)
        const char* __restrict__ const ab = g.add_base;
        const uint32_t* __restrict__ const ai = g.add_index;
        const uint32_t cnt = *g.add_count;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            uint32_t add_row[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm + 32 * i + 8 * (r >> 2) + 4 * hl + (r & 3);
                add_row[r] = (uint32_t)m < cnt ? ai[m] : 0u;
            }
            float addv[16][NJ];
#pragma unroll
            for (int r = 0; r < 16; ++r)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    addv[r][j] = load1(ab + (int64_t)add_row[r] * g.add_pitch, n0 + wn + 32 * j + cl, g.add_etype);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm + 32 * i + 8 * (r >> 2) + 4 * hl + (r & 3);
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    Cr[(size_t)m * g.ldc + n0 + wn + 32 * j + cl] = acc[i][j][r] + addv[r][j];
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm + 32 * i + 8 * (r >> 2) + 4 * hl + (r & 3);
#pragma unroll
            for (int j = 0; j < NJ; ++j) Cr[(size_t)m * g.ldc + n0 + wn + 32 * j + cl] = acc[i][j][r];
        }
}

bool gemm_nt_bf16_ok(int M, int N, int K) { return M % 128 == 0 && N % 128 == 0 && K % GB_K == 0; }

// The tile and the contraction split of a product, from the workgroups that will find work
// (`live`: a device-side limit on rows or columns is taken to leave half the tiles, one on the
// contraction half the splits).  Without a split where some tile makes two live workgroups per
// CU: the largest such tile.  Else, where the caller has room for partial products, the largest
// tile that reaches one live workgroup per CU with at most 16 splits (powers of two, at least
// 256 columns each) and the fewest splits that do; else the smallest tile, unsplit.
// Measured on the 8192 x 2048 x 512 workload with 768 features (us per step, the product's
// kernel group): d q 128 x 64 unsplit 60.7 against 66.0 (128 x 128, 2 splits); d tails 8 splits
// 60 at any tile against 64.5 (16) and 72.9 (4); hidden 64 x 64 28.0 against 35.3 (128 x 128);
// d W 128 x 64 with 16 splits 31.1 against 33.0 (128 x 128) and 37.4 (64 x 64).
struct GemmPlan { int tm, tn, ks; };
static GemmPlan gemm_nt_bf16_plan(int M, int N, int K, int batches, bool mn_limited, bool k_limited, bool may_split) {
    const int cand[3][2] = {{128, 128}, {128, 64}, {64, 64}};
    auto tiles = [&](const int* t) { return (long)(M / t[0]) * (N / t[1]) * batches / (mn_limited ? 2 : 1); };
    for (const auto& t : cand)
        if (tiles(t) >= 512) return {t[0], t[1], 1};
    if (may_split) {
        const int k_div = k_limited ? 2 : 1;
        for (const auto& t : cand) {
            GemmPlan p = {t[0], t[1], 1};
            auto can_double = [&]() { return p.ks < 16 && K % (2 * p.ks * GB_K) == 0 && K / (2 * p.ks) >= 256; };
            while (tiles(t) * p.ks / k_div < 256 && can_double()) p.ks *= 2;
            if (tiles(t) * p.ks / k_div >= 256) return p;
        }
    }
    return {64, 64, 1};
}

// Room for the partial products of a split contraction: the largest split any combination of
// limits may choose (batches * ksplit * M * N floats).
int gemm_nt_bf16_ksplit(int M, int N, int K, int batches) {
    int ks = 1;
    for (int f = 0; f < 4; ++f) ks = std::max(ks, gemm_nt_bf16_plan(M, N, K, batches, f & 1, f & 2, true).ks);
    return ks;
}

// out[b][i] = sum over s of part[b][s][i], in order (n % 4 == 0); blockIdx.y = b
__global__ __launch_bounds__(256) void k_sum_split_batches(const float* __restrict__ part, int ns, int64_t n,
                                                           float* __restrict__ out, int64_t out_batch) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    const float* p = part + (size_t)blockIdx.y * ns * n + i;
    float4 acc = *reinterpret_cast<const float4*>(p);
    for (int s = 1; s < ns; ++s) acc = f4add(acc, *reinterpret_cast<const float4*>(p + (size_t)s * n));
    *reinterpret_cast<float4*>(out + (size_t)blockIdx.y * out_batch + i) = acc;
}

// With g.part set the contraction may be split (gemm_nt_bf16_ksplit); the partial
// products are added in split order.  Splitting needs ldc == N (dense partials).
void launch_gemm_nt_bf16(const GemmNT& g0, hipStream_t stream) {
    GemmNT g = g0;
    const GemmPlan t = gemm_nt_bf16_plan(g.M, g.N, g.K, g.batches, g.m_limit || g.n_limit, g.k_limit != nullptr,
                                         g.part && g.ldc == g.N && !g.add_base);
    g.ksplit = t.ks;
    const dim3 grid = tile_grid(g.N / t.tn, g.M / t.tm, g.batches * g.ksplit);
#define KGE_GEMM_TILE(AK_, BK_)                                                                              \
    do {                                                                                                     \
        if (t.tm == 128 && t.tn == 128) hipLaunchKernelGGL((k_gemm_nt_bf16<AK_, BK_, 128, 128>), grid, dim3(256), 0, stream, g); \
        else if (t.tm == 128) hipLaunchKernelGGL((k_gemm_nt_bf16<AK_, BK_, 128, 64>), grid, dim3(256), 0, stream, g);           \
        else hipLaunchKernelGGL((k_gemm_nt_bf16<AK_, BK_, 64, 64>), grid, dim3(256), 0, stream, g);          \
    } while (0)
    if (g.a_kmajor && g.b_kmajor == 2) KGE_GEMM_TILE(true, 2);
    else if (g.a_kmajor && g.b_kmajor) KGE_GEMM_TILE(true, 1);
    else if (g.a_kmajor) KGE_GEMM_TILE(true, 0);
    else if (g.b_kmajor == 2) KGE_GEMM_TILE(false, 2);
    else if (g.b_kmajor) KGE_GEMM_TILE(false, 1);
    else KGE_GEMM_TILE(false, 0);
#undef KGE_GEMM_TILE
    if (g.ksplit > 1) {
        const int64_t n = (int64_t)g.M * g.N;
        hipLaunchKernelGGL(k_sum_split_batches, dim3((unsigned)((n / 4 + 255) / 256), g.batches), dim3(256), 0,
                           stream, g.part, g.ksplit, n, g.C, g.c_batch);
    }
}

// --------------------------------------------------------------------------
// row-wise losses: softmax cross entropy with the sampling correction
// (src/poplar_kge.cpp:638-652) and logsigmoid with self-adversarial negative
// weights (src/poplar_kge.cpp:623-633).  One wave per (block, positive).

__global__ __launch_bounds__(256) void k_loss_rows(ScoreShape sh, const uint32_t* __restrict__ clabel,
                                                   float* __restrict__ coef,
                                                   const float* __restrict__ dist,
                                                   float* __restrict__ loss_part,
                                                   uint16_t* __restrict__ coef16, int keep_f32) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);  // d*B + b
    if (row >= sh.S * sh.B) return;
    const int T = sh.T;
    float* s = coef + (size_t)row * T;
    uint16_t* s16 = coef16 ? coef16 + (size_t)row * T : nullptr;  // bfloat16 copy for the matrix cores
    const float* dr = dist ? dist + (size_t)row * T : nullptr;
    const uint32_t label = clabel[row];
    // merged tails: the block's live columns and how many tail positions each stands for.  Column j
    // of multiplicity m holds m negatives, or the label's position and m - 1 negatives; the sums
    // below run over positions, so a column enters them m times (src/poplar_kge.cpp:615-652).
    const int blk = row / sh.B;
    const int TL = tail_limit(sh.tcount, blk, T, sh.tpad);
    const float* mu = sh.tmult ? sh.tmult + (size_t)blk * T : nullptr;
    float loss = 0.f;
    if (sh.loss_fn == LOSS_SOFTMAX && (T & 3) == 0 && T <= 2048) {
        // the row stays in registers (up to eight float4 per lane): one read, one write
        const float corr = sh.softmax_correction;
        constexpr int NV = 8;
        floatx4 z[NV], m[NV];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int t = 4 * lane + 256 * i;
            if (t < TL) {
                z[i] = *reinterpret_cast<const floatx4*>(s + t);
                m[i] = mu ? *reinterpret_cast<const floatx4*>(mu + t) : floatx4{1.f, 1.f, 1.f, 1.f};
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const bool pos = (uint32_t)(t + x) == label;
                    if (m[i][x] == 0.f) z[i][x] = -INFINITY;  // no position holds this column
                    if (!pos || m[i][x] > 1.f) mx = fmaxf(mx, z[i][x] + corr);
                    if (pos) mx = fmaxf(mx, z[i][x]);
                }
            }
        }
        mx = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (4 * lane + 256 * i < TL)
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const bool pos = (uint32_t)(4 * lane + 256 * i + x) == label;
                    const float neg = m[i][x] - (pos ? 1.f : 0.f);
                    if (neg > 0.f) sum += neg * __expf(z[i][x] + corr - mx);
                    if (pos) sum += __expf(z[i][x] - mx);
                }
        sum = wave_sum(sum);
        const float lse = mx + logf(sum);
        const float inv_norm = 1.f / ((float)sh.S * (float)sh.B);
        const float gs = inv_norm * sh.loss_scale;
        const float sgn = score_is_distance_value(sh.score_fn) ? 1.f : -1.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int t = 4 * lane + 256 * i;
            if (t < TL) {
                floatx4 c;
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const bool pos = (uint32_t)(t + x) == label;
                    const float neg = m[i][x] - (pos ? 1.f : 0.f);
                    float g = neg > 0.f ? neg * __expf(z[i][x] + corr - lse) : 0.f;
                    if (pos) {
                        loss = -(z[i][x] - lse) * inv_norm;
                        g += __expf(z[i][x] - lse) - 1.f;
                    }
                    c[x] = sgn * g * gs;
                }
                if (dr) {
                    const floatx4 dv = *reinterpret_cast<const floatx4*>(dr + t);
#pragma unroll
                    for (int x = 0; x < 4; ++x) c[x] = dv[x] != 0.f ? c[x] / dv[x] : 0.f;
                }
                if (keep_f32) *reinterpret_cast<floatx4*>(s + t) = c;
                if (s16) {
                    uint2 raw;
                    raw.x = (uint32_t)f32_to_bf16(c.x) | ((uint32_t)f32_to_bf16(c.y) << 16);
                    raw.y = (uint32_t)f32_to_bf16(c.z) | ((uint32_t)f32_to_bf16(c.w) << 16);
                    *reinterpret_cast<uint2*>(s16 + t) = raw;
                }
            }
        }
    } else if (sh.loss_fn == LOSS_SOFTMAX) {
        const float corr = sh.softmax_correction;
        float mx = -INFINITY;
        for (int t = lane; t < TL; t += 64) {
            const bool pos = (uint32_t)t == label;
            const float m = mu ? mu[t] : 1.f;
            if (m - (pos ? 1.f : 0.f) > 0.f) mx = fmaxf(mx, s[t] + corr);
            if (pos) mx = fmaxf(mx, s[t]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
        for (int t = lane; t < TL; t += 64) {
            const bool pos = (uint32_t)t == label;
            const float neg = (mu ? mu[t] : 1.f) - (pos ? 1.f : 0.f);
            if (neg > 0.f) sum += neg * expf(s[t] + corr - mx);
            if (pos) sum += expf(s[t] - mx);
        }
        sum = wave_sum(sum);
        const float lse = mx + logf(sum);
        const float inv_norm = 1.f / ((float)sh.S * (float)sh.B);
        for (int t = lane; t < TL; t += 64) {
            const bool pos = (uint32_t)t == label;
            const float neg = (mu ? mu[t] : 1.f) - (pos ? 1.f : 0.f);
            float g = neg > 0.f ? neg * expf(s[t] + corr - lse) : 0.f;
            if (pos) {
                loss = -(s[t] - lse) * inv_norm;
                g += expf(s[t] - lse) - 1.f;
            }
            const float ds = g * inv_norm * sh.loss_scale;
            float c = score_is_distance_value(sh.score_fn) ? ds : -ds;
            if (dr) c = dr[t] != 0.f ? c / dr[t] : 0.f;
            s[t] = c;
            if (s16) s16[t] = f32_to_bf16(c);
        }
    } else {
        const float adv = sh.negative_adversarial_scale;
        const float Tn = (float)T;
        const float w_pos = 0.5f * Tn, w_neg = (0.5f * Tn) / (float)(T - 1);
        const float inv_norm = 1.f / ((float)sh.S * (float)sh.B * Tn);
        float mx = -INFINITY, sum = 1.f;
        if (adv > 0.f) {
            // softmax over the positions of adv * score, the label's position pushed down by 10000
            for (int t = lane; t < TL; t += 64) {
                const bool pos = (uint32_t)t == label;
                const float m = mu ? mu[t] : 1.f;
                if (m - (pos ? 1.f : 0.f) > 0.f) mx = fmaxf(mx, adv * s[t]);
                if (pos) mx = fmaxf(mx, adv * s[t] - 10000.f);
            }
            mx = wave_max(mx);
            sum = 0.f;
            for (int t = lane; t < TL; t += 64) {
                const bool pos = (uint32_t)t == label;
                const float neg = (mu ? mu[t] : 1.f) - (pos ? 1.f : 0.f);
                if (neg > 0.f) sum += neg * expf(adv * s[t] - mx);
                if (pos) sum += expf(adv * s[t] - 10000.f - mx);
            }
            sum = wave_sum(sum);
        }
        for (int t = lane; t < TL; t += 64) {
            const bool pos = (uint32_t)t == label;
            const float neg = (mu ? mu[t] : 1.f) - (pos ? 1.f : 0.f);
            const float sc = s[t];
            float wl = w_pos, wn = w_neg;  // weight of the label's position, of one negative position
            if (adv > 0.f) {
                wl *= 1.f + (Tn - 1.f) * (expf(adv * sc - 10000.f - mx) / sum);
                wn *= (Tn - 1.f) * (expf(adv * sc - mx) / sum);
            }
            float ds = 0.f;
            if (pos) {
                loss -= wl * log_sigmoid(sc) * inv_norm;
                ds -= wl * log_sigmoid_grad(sc);
            }
            if (neg > 0.f) {
                loss -= neg * wn * log_sigmoid(-sc) * inv_norm;
                ds += neg * wn * log_sigmoid_grad(-sc);
            }
            ds *= inv_norm * sh.loss_scale;
            float c = score_is_distance_value(sh.score_fn) ? ds : -ds;
            if (dr) c = dr[t] != 0.f ? c / dr[t] : 0.f;
            s[t] = c;
            if (s16) s16[t] = f32_to_bf16(c);
        }
    }
    loss = wave_sum(loss);
    if (lane == 0) loss_part[row] = loss;
}

void launch_loss_rows(const ScoreShape& sh, const uint32_t* clabel, float* coef, const float* dist,
                      float* loss_part, uint16_t* coef16, hipStream_t stream, bool keep_f32) {
    const int rows = sh.S * sh.B;
    const bool l2 = sh.score_fn != SCORE_DISTMULT && sh.dist_fn == DIST_L2;
    hipLaunchKernelGGL(k_loss_rows, dim3((rows + 3) / 4), dim3(256), 0, stream, sh, clabel, coef,
                       l2 ? dist : nullptr, loss_part, coef16, (coef16 && !keep_f32) ? 0 : 1);
}

// --------------------------------------------------------------------------
// The loss functions as stand-alone device ops (pag::ops::logSigmoid, src/pag/pag.cpp:888-910;
// pag::ops::logSoftmax, :841-864), evaluated by the same device functions the step's kernels call.

// form 0: log_sigmoid / log_sigmoid_grad as k_loss_rows calls them; form 1: log_sigmoid_both,
// the one-exponential form of the scoring epilogues
__global__ __launch_bounds__(256) void k_log_sigmoid(const float* __restrict__ x, const float* __restrict__ dy,
                                                     float* __restrict__ y, float* __restrict__ dx, int64_t n,
                                                     int form) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float v, g;
    if (form) log_sigmoid_both(x[i], v, g);
    else { v = log_sigmoid(x[i]); g = log_sigmoid_grad(x[i]); }
    if (y) y[i] = v;
    if (dx) dx[i] = (dy ? dy[i] : 1.f) * g;
}
void launch_log_sigmoid(const float* x, const float* dy, float* y, float* dx, int64_t n, int form,
                        hipStream_t stream) {
    if (n <= 0) return;
    hipLaunchKernelGGL(k_log_sigmoid, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, dy, y, dx, n, form);
}

// One wave per row.  Forward: y = x - max - log(sum exp(x - max)) (the reduction k_loss_rows makes
// for the softmax loss).  Backward (dy given, `x` holds y): dx = dy - exp(y) * sum(dy)
// (src/pag/pag.cpp:853-859).
__global__ __launch_bounds__(256) void k_log_softmax(const float* __restrict__ x, const float* __restrict__ dy,
                                                     float* __restrict__ out, int64_t rows, int64_t cols) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* xr = x + row * cols;
    float* o = out + row * cols;
    if (!dy) {
        float mx = -INFINITY;
        for (int64_t t = lane; t < cols; t += 64) mx = fmaxf(mx, xr[t]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int64_t t = lane; t < cols; t += 64) sum += expf(xr[t] - mx);
        sum = wave_sum(sum);
        const float lse = mx + logf(sum);
        for (int64_t t = lane; t < cols; t += 64) o[t] = xr[t] - lse;
    } else {
        const float* dr = dy + row * cols;
        float sum = 0.f;
        for (int64_t t = lane; t < cols; t += 64) sum += dr[t];
        sum = wave_sum(sum);
        for (int64_t t = lane; t < cols; t += 64) o[t] = dr[t] - expf(xr[t]) * sum;
    }
}
void launch_log_softmax(const float* x, const float* dy, float* out, int64_t rows, int64_t cols,
                        hipStream_t stream) {
    if (rows <= 0 || cols <= 0) return;
    hipLaunchKernelGGL(k_log_softmax, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, x, dy, out, rows, cols);
}

// --------------------------------------------------------------------------
// predict: running top-k over a stream of score chunks
// (TopKCollector, src/poplar_kge.cpp:743-809).  One workgroup per query keeps
// its n_best (score, index) pairs sorted by (score descending, index
// ascending).  New scores are compared with the current n_best-th score 16384
// at a time (64 per thread, all loads in flight together); the few that beat it
// are collected in LDS (in any order) and merged by rank: every element of
// (current best, candidates) counts the candidates that come before it, a
// candidate also finds its place among the sorted best by binary search, and
// the elements whose rank is below n_best are written to that place.  The
// order is total on distinct rows, so the result does not depend on the order
// of collection, and ties resolve to the lower index whatever the chunking.
// A pass with more than 1024 candidates is redone 1024 scores at a time.

constexpr int TK_BLOCK = 1024;  // most n_best, and the candidate list's capacity
constexpr int TK_SPAN = 16384;

DEVINL bool topk_before(float sa, uint32_t ia, float sb, uint32_t ib) {
    return sa > sb || (sa == sb && ia < ib);
}

__global__ __launch_bounds__(256) void k_topk_merge(const float* __restrict__ scores, int64_t ld,
                                                    int n_valid, uint32_t first_index, int n_best,
                                                    float* __restrict__ best_score,
                                                    uint32_t* __restrict__ best_index) {
    __shared__ __attribute__((aligned(16))) float cand_s[TK_BLOCK];
    __shared__ __attribute__((aligned(16))) uint32_t cand_i[TK_BLOCK];
    __shared__ float cur_s[TK_BLOCK], next_s[TK_BLOCK];
    __shared__ uint32_t cur_i[TK_BLOCK], next_i[TK_BLOCK];
    // candidate counters of three consecutive passes: the one of the pass after this one is cleared
    // before this pass's barrier, when every thread has read its previous value (a pass ago)
    __shared__ int n_cand[3];
    const int q = blockIdx.x, tid = threadIdx.x;
    const float* row = scores + (size_t)q * ld;
    float* bs = best_score + (size_t)q * n_best;
    uint32_t* bi = best_index + (size_t)q * n_best;
    for (int i = tid; i < n_best; i += 256) {
        cur_s[i] = bs[i];
        cur_i[i] = bi[i];
    }
    if (tid == 0) n_cand[0] = n_cand[1] = 0;
    __syncthreads();
    bool changed = false;
    int pass = 0;
    // Scores per pass: TK_SPAN, all loads of a pass in flight together.  While the list still holds
    // its initial entries (row 0, which never competes) every score is a candidate, so a sweep
    // starts with 256 and doubles: each pass then brings about n_best * ln 2 candidates.
    int piece = cur_i[n_best - 1] == 0u ? 256 : TK_SPAN;
    {
        for (int base = 0; base < n_valid;) {
            const int end = min(n_valid, base + piece);
            const float kth = cur_s[n_best - 1];
            int* counter = &n_cand[pass % 3];
            if (tid == 0) n_cand[(pass + 1) % 3] = 0;
            ++pass;
            constexpr int NV = TK_SPAN / 1024;
            float4 v[NV];
#pragma unroll
            for (int j = 0; j < NV; ++j) {  // rows are 16-byte aligned and hold a multiple of 4 scores
                const int i = base + 1024 * j + tid * 4;
                v[j] = i < end ? *reinterpret_cast<const float4*>(row + i) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
            }
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const float* vv = &v[j].x;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = base + 1024 * j + tid * 4 + e;
                    if (i < end && vv[e] > kth) {  // false for NaN
                        const int slot = atomicAdd(counter, 1);
                        if (slot < TK_BLOCK) {
                            cand_s[slot] = vv[e];
                            cand_i[slot] = first_index + (uint32_t)i;
                        }
                    }
                }
            }
            __syncthreads();
            const int c = *counter;  // the same for every thread: all branches below are uniform
            if (c > TK_BLOCK) {  // more than the list holds: the same scores again, TK_BLOCK at a time
                piece = TK_BLOCK;
                continue;
            }
            base = end;
            piece = min(2 * piece, TK_SPAN);
            if (c == 0) continue;
            changed = true;
            // candidates padded to whole groups of four with entries that come before nothing
            for (int x = c + tid; x < ((c + 3) & ~3); x += 256) {
                cand_s[x] = -INFINITY;
                cand_i[x] = 0xffffffffu;
            }
            __syncthreads();
            // a thread's elements: candidates tid + 256 m (m < 4), current best tid + 256 (m - 4)
            constexpr int PER = TK_BLOCK / 256;
            float es[2 * PER];
            uint32_t ei[2 * PER];
            int r[2 * PER];
#pragma unroll
            for (int m = 0; m < PER; ++m) {
                const int e = tid + 256 * m;
                es[m] = e < c ? cand_s[e] : -INFINITY;
                ei[m] = e < c ? cand_i[e] : 0xffffffffu;
                int lo = 0, hi = e < c ? n_best : 0;
                while (lo < hi) {  // entries of the sorted best that come before this candidate
                    const int mid = (lo + hi) >> 1;
                    if (topk_before(cur_s[mid], cur_i[mid], es[m], ei[m])) lo = mid + 1;
                    else hi = mid;
                }
                r[m] = e < c ? lo : n_best;
                es[PER + m] = e < n_best ? cur_s[e] : -INFINITY;
                ei[PER + m] = e < n_best ? cur_i[e] : 0xffffffffu;
                r[PER + m] = e < n_best ? e : n_best;
            }
            // every element counts the candidates before it: four candidates per LDS read (the same
            // address for all lanes), up to eight elements per lane against them
            for (int x = 0; x < c; x += 4) {
                const float4 s4 = *reinterpret_cast<const float4*>(&cand_s[x]);
                const uint4 i4 = *reinterpret_cast<const uint4*>(&cand_i[x]);
#pragma unroll
                for (int m = 0; m < 2 * PER; ++m) {
                    const bool live = m < PER ? 256 * m < c : 256 * (m - PER) < n_best;  // uniform
                    if (!live) continue;
                    r[m] += (topk_before(s4.x, i4.x, es[m], ei[m]) ? 1 : 0) + (topk_before(s4.y, i4.y, es[m], ei[m]) ? 1 : 0) +
                            (topk_before(s4.z, i4.z, es[m], ei[m]) ? 1 : 0) + (topk_before(s4.w, i4.w, es[m], ei[m]) ? 1 : 0);
                }
            }
#pragma unroll
            for (int m = 0; m < 2 * PER; ++m)
                if (r[m] < n_best) {
                    next_s[r[m]] = es[m];
                    next_i[r[m]] = ei[m];
                }
            __syncthreads();
            for (int i = tid; i < n_best; i += 256) {
                cur_s[i] = next_s[i];
                cur_i[i] = next_i[i];
            }
            __syncthreads();
        }
    }
    if (changed)
        for (int i = tid; i < n_best; i += 256) {
            bs[i] = cur_s[i];
            bi[i] = cur_i[i];
        }
}

void launch_topk_merge(const float* scores, int64_t ld, int n_queries, int n_valid, uint32_t first_index,
                       int n_best, float* best_score, uint32_t* best_index, hipStream_t stream) {
    if ((ld & 3) || n_valid > ld || ((uintptr_t)scores & 15)) throw std::invalid_argument("top-k merge: score rows must be 16-byte aligned");
    hipLaunchKernelGGL(k_topk_merge, dim3(n_queries), dim3(256), 0, stream, scores, ld, n_valid, first_index,
                       n_best, best_score, best_index);
}

// out[i] = base + i for i < n_live, 0 (the padding row) after that
__global__ __launch_bounds__(256) void k_row_range(uint32_t base, int n_live, int n, uint32_t* __restrict__ out) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = i < n_live ? base + (uint32_t)i : 0u;
}
void launch_row_range(uint32_t base, int n_live, int n, uint32_t* out, hipStream_t stream) {
    hipLaunchKernelGGL(k_row_range, dim3((n + 255) / 256), dim3(256), 0, stream, base, n_live, n, out);
}

// --------------------------------------------------------------------------
// segmented reduction + Adam

// One gradient contribution (row c of the contribution-gradient matrix), four
// columns from k, with the DistMult product rule applied on load.
template <bool XF>  // XF: the ComplEx / RotatE transforms (3 .. 6) are compiled in
DEVINL float4 load_contrib(const ContribSrc& cs, uint32_t c, int k, int Dp) {
    float4 g = *reinterpret_cast<const float4*>(cs.grad + (size_t)c * Dp + k);
    if (XF && cs.transform >= 5) {
        // RotatE: the predicted tail is (h_re, h_im) rotated by the phases.  Entity plan: the
        // gradient rotated back.  Relation plan: the phases' gradient, formed in float16 as the
        // reference's float16 sine / cosine backward ops form it (src/pag/pag.cpp:552-637),
        // in columns [0, half); zero above.
        if (c < (uint32_t)cs.n_head) {
            const float* gr = cs.grad + (size_t)c * Dp;
            const float* rr = cs.rel + (size_t)cs.crel[c] * Dp;
            const char* er = row_ptr(cs.ent, c);
            float* gg = &g.x;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int kk = k + x;
                if (kk >= 2 * cs.half) { gg[x] = 0.f; continue; }
                const int kq = kk < cs.half ? kk : kk - cs.half;
                const float th = (float)(_Float16)rr[kq];
                const _Float16 sn = (_Float16)sinf(th), cs16 = (_Float16)cosf(th);
                const float g_re = gr[kq], g_im = gr[kq + cs.half];
                if (cs.transform == 5) {
                    gg[x] = kk < cs.half ? g_re * (float)cs16 + g_im * (float)sn
                                         : g_im * (float)cs16 - g_re * (float)sn;
                } else if (kk < cs.half) {
                    const float h_re = load1(er, kq, cs.ent.etype), h_im = load1(er, kq + cs.half, cs.ent.etype);
                    const _Float16 g_sin = (_Float16)(-g_re * h_im + g_im * h_re);
                    const _Float16 g_cos = (_Float16)(g_re * h_re + g_im * h_im);
                    const _Float16 from_cos = -g_cos * sn, from_sin = g_sin * cs16;
                    gg[x] = (float)(_Float16)(from_cos + from_sin);
                } else {
                    gg[x] = 0.f;
                }
            }
        }
    } else if (XF && cs.transform >= 3) {
        // ComplEx: the predicted tail is the complex product h r, so the head's gradient is
        // g conj(r) and the relation's g conj(h) (column kk pairs with kk +- half):
        //   re: g_re o_re + g_im o_im      im: g_im o_re - g_re o_im      (o = r or h)
        if (c < (uint32_t)cs.n_head) {
            const float* gr = cs.grad + (size_t)c * Dp;
            const float* rr = cs.rel + (size_t)cs.crel[c] * Dp;
            const char* er = row_ptr(cs.ent, c);
            float* gg = &g.x;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int kk = k + x;
                if (kk >= 2 * cs.half) { gg[x] = 0.f; continue; }
                const int pp = kk < cs.half ? kk + cs.half : kk - cs.half;
                const float o_k = cs.transform == 3 ? rr[kk] : load1(er, kk, cs.ent.etype);
                const float o_p = cs.transform == 3 ? rr[pp] : load1(er, pp, cs.ent.etype);
                const float g_p = gr[pp];
                gg[x] = kk < cs.half ? gg[x] * o_k + g_p * o_p : gg[x] * o_p - g_p * o_k;
            }
        }
    } else if (cs.transform == 1) {
        if (c < (uint32_t)cs.n_head)
            g = f4mul(g, *reinterpret_cast<const float4*>(cs.rel + (size_t)cs.crel[c] * Dp + k));
    } else if (cs.transform == 2) {
        g = f4mul(g, load4(row_ptr(cs.ent, c), k, cs.ent));
    }
    return g;
}

// Ordered sum of the contributions at sorted positions [pos, pos + n), columns
// k..k+3: eight independent row loads in flight, added in position order.
// Must be called by every lane of the wave (the item indices travel by
// shuffle); lanes with `active` false load nothing and return zero.
template <int NB, bool XF>
DEVINL float4 sum_contribs(const ContribSrc& cs, uint32_t pos, uint32_t n, int k, int Dp, int lane,
                           bool active) {
    float4 acc = make_float4(0, 0, 0, 0);
    for (uint32_t j = 0; j < n; j += NB) {
        const uint32_t mine = (j + (lane & (NB - 1)) < n) ? cs.sorted_item[pos + j + (lane & (NB - 1))] : 0u;
        float4 v[NB];
#pragma unroll
        for (int x = 0; x < NB; ++x) {
            const uint32_t c = __shfl(mine, x, 64);
            v[x] = (active && j + x < n) ? load_contrib<XF>(cs, c, k, Dp) : make_float4(0, 0, 0, 0);
        }
#pragma unroll
        for (int x = 0; x < NB; ++x) acc = f4add(acc, v[x]);
    }
    return acc;
}

// First level for rows with many contributions: one workgroup per chunk, each
// of its NW waves sums an NW-th of the chunk, the NW sums are added in wave order.
// NW = 16 serves chunks of up to 256 contributions with the same two rounds of
// eight loads per wave that NW = 4 needs for 64: four times fewer partials for
// the second level to walk through.
template <int NW, bool XF>
__global__ __launch_bounds__(NW * 64) void k_reduce_chunks(ReduceArgs a0, ReduceArgs a1) {
    __shared__ __attribute__((aligned(16))) float part[NW - 1][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // two reductions share the launch: blocks [0, a0.max_chunks * slabs) serve the first; a
    // workgroup takes one slab of 256 columns of one chunk (rows wider than 256 columns: the
    // slabs' chains of dependent loads run side by side instead of one after the other)
    const int slabs = (max(a0.Dp, a1.Dp) + 255) / 256;
    const int b = blockIdx.x / slabs, slab = blockIdx.x - b * slabs;
    const bool second = b >= a0.max_chunks;
    const ReduceArgs& a = second ? a1 : a0;
    const int q = second ? b - a0.max_chunks : b;
    // fetched together with the chunk count (entries past it are stale but inside the arrays):
    // one round trip less in front of every chunk
    const uint32_t pos = a.chunk_pos[q], len = a.chunk_len[q];
    if (q >= (int)a.counts[1]) return;
    const int Dp = a.Dp;
    if (Dp & 3) {  // unaligned rows (stand-alone scatter-add on arbitrary widths): wave 0 only
        if (wave == 0)
            for (int k = slab * 256 + lane; k < min(Dp, (slab + 1) * 256); k += 64) {
                float acc = 0.f;
                for (uint32_t j = 0; j < len; ++j)
                    acc += a.src.grad[(size_t)a.src.sorted_item[pos + j] * Dp + k];
                a.partial[(size_t)q * Dp + k] = acc;
            }
        return;
    }
    const uint32_t share = (len + NW - 1) / NW;
    const uint32_t w0 = min(len, wave * share), w1 = min(len, w0 + share);
    const int k = slab * 256 + lane * 4;
    // sixteen loads in flight: a wave's share of a 64-item chunk in one round (same order of
    // additions as any other round size)
    float4 acc = sum_contribs<16, XF>(a.src, pos + w0, w1 - w0, k, Dp, lane, k < Dp);
    if (wave > 0) *reinterpret_cast<float4*>(&part[wave - 1][lane * 4]) = acc;
    __syncthreads();
    if (wave == 0 && k < Dp) {
#pragma unroll
        for (int w = 0; w < NW - 1; ++w) acc = f4add(acc, *reinterpret_cast<const float4*>(&part[w][lane * 4]));
        *reinterpret_cast<float4*>(a.partial + (size_t)q * Dp + k) = acc;
    }
}

static void launch_reduce_kernel(const ReduceArgs& a0, const ReduceArgs& a1, hipStream_t stream) {
    const int n = (a0.max_chunks + a1.max_chunks) * ((std::max(a0.Dp, a1.Dp) + 255) / 256);
    if (n == 0) return;
    const bool xf = (a0.max_chunks && a0.src.transform >= 3) || (a1.max_chunks && a1.src.transform >= 3);
    if (std::max(a0.chunk, a1.chunk) > 64) {
        if (xf) hipLaunchKernelGGL((k_reduce_chunks<16, true>), dim3(n), dim3(1024), 0, stream, a0, a1);
        else hipLaunchKernelGGL((k_reduce_chunks<16, false>), dim3(n), dim3(1024), 0, stream, a0, a1);
    } else {
        if (xf) hipLaunchKernelGGL((k_reduce_chunks<4, true>), dim3(n), dim3(256), 0, stream, a0, a1);
        else hipLaunchKernelGGL((k_reduce_chunks<4, false>), dim3(n), dim3(256), 0, stream, a0, a1);
    }
}
void launch_reduce_chunks(const ReduceArgs& a, hipStream_t stream) {
    ReduceArgs none = a;
    none.max_chunks = 0;
    launch_reduce_kernel(a, none, stream);
}
void launch_reduce_chunks2(const ReduceArgs& a0, const ReduceArgs& a1, hipStream_t stream) {
    launch_reduce_kernel(a0, a1, stream);
}

// fr::nn::adam (src/fructose/frnn.cpp:74-89) on one float4
DEVINL void adam4(float4& p, float4& m, float4& v, float4 g, const AdamArgs& a, float alpha) {
    float* pp = &p.x; float* mm = &m.x; float* vv = &v.x; const float* gg = &g.x;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        float vi = vv[x];
        if (a.v_is_sqrt) vi = vi * vi;
        const float mi = a.beta_m * mm[x] + a.one_minus_beta_m * gg[x];
        vi = a.beta_v * vi + a.one_minus_beta_v * gg[x] * gg[x];
        pp[x] = pp[x] - alpha * (mi / (sqrtf(vi) + a.epsilon) + a.weight_decay * pp[x]);
        mm[x] = mi;
        vv[x] = a.v_is_sqrt ? sqrtf(vi) : vi;
    }
}

// One wave per distinct row: gather its gradient (directly from its few
// contributions, or from its chunk partials), Adam, write the row back.
// MF32: both moments float32 (the usual layout), accessed as plain 16-byte words
// A wave's life is a chain of dependent loads (plan entry, item list, contribution rows and the
// row itself, stores): what the kernel gets through is the number of resident waves over that
// chain's length, so the plain form is compiled for eight waves per SIMD (four contribution
// loads in flight instead of eight buy the registers).
template <bool MF32, bool XF>
DEVINL void adam_rows_body(const AdamArgs& a0, const AdamArgs& a1) {
    const int lane = threadIdx.x & 63;
    // two tables share the launch: blocks [0, ceil(a0.max_rows * slabs / 4)) serve the first; a
    // wave takes one slab of 256 columns of one row
    const int slabs = (max(a0.Dp, a1.Dp) + 255) / 256;
    const int blocks0 = (a0.max_rows * slabs + 3) / 4;
    const bool second = (int)blockIdx.x >= blocks0;
    const AdamArgs& a = second ? a1 : a0;
    const int g = (second ? blockIdx.x - blocks0 : blockIdx.x) * 4 + (threadIdx.x >> 6);
    const int u = g / slabs, slab = g - u * slabs;
    // the row's plan entries are fetched together with the row count (entries past it are stale
    // but inside the arrays): one round trip less in front of every row
    const int uc = min(u, a.max_rows - 1);
    const uint32_t key = a.uniq_key[uc];
    uint32_t q0 = 0, q1 = 0, pos = 0, n_real = 0;
    if (!a.grad_direct) {
        q0 = a.chunk_off[uc]; q1 = a.chunk_off[uc + 1];
        pos = a.seg_start[uc]; n_real = a.seg_real[uc];
    }
    if (u >= (int)a.counts[0]) return;
    const float alpha = a.alpha[a.rows_per_alpha ? key / a.rows_per_alpha : 0u];
    const int Dp = a.Dp;
    char* prow = a.p_base + (int64_t)key * a.pitch;
    char* mrow = a.m_base + (int64_t)key * a.pitch;
    char* vrow = a.v_base + (int64_t)key * a.pitch;
    {
        const int k = slab * 256 + lane * 4;
        const bool active = k < Dp;
        float4 g = make_float4(0, 0, 0, 0);
        if (!a.grad_direct && q1 == q0 && n_real)  // wave-uniform: all lanes take part in the shuffles
            g = sum_contribs<XF ? 8 : 4, XF>(a.src, pos, n_real, k, Dp, lane, active);
        if (!active) return;
        float4 p = load4(prow, k, a.p_etype);
        float4 m, v;
        if constexpr (MF32) {
            m = *reinterpret_cast<const float4*>(mrow + (size_t)k * 4);
            v = *reinterpret_cast<const float4*>(vrow + (size_t)k * 4);
        } else {
            m = load4(mrow, k, a.m_etype);
            v = load4(vrow, k, a.m_etype);
        }
        if (a.grad_direct) {
            g = *reinterpret_cast<const float4*>(a.grad_direct + (size_t)u * Dp + k);
        } else if (q1 > q0) {
            constexpr int NP = XF ? 8 : 4;  // partial sums in flight
            for (uint32_t q = q0; q < q1; q += NP) {
                float4 t[NP];
#pragma unroll
                for (int x = 0; x < NP; ++x)
                    t[x] = (q + x < q1) ? *reinterpret_cast<const float4*>(a.partial + (size_t)(q + x) * Dp + k)
                                        : make_float4(0, 0, 0, 0);
#pragma unroll
                for (int x = 0; x < NP; ++x) g = f4add(g, t[x]);
            }
        }
        if (a.grad_out) {
            float4 go = g;
            if (a.grad_out_add) go = f4add(go, *reinterpret_cast<const float4*>(a.grad_out_add + (size_t)u * Dp + k));
            *reinterpret_cast<float4*>(a.grad_out + (size_t)u * Dp + k) = go;
        }
        if (a.no_update) return;
        if (a.grad_add) g = f4add(g, *reinterpret_cast<const float4*>(a.grad_add + (size_t)u * Dp + k));
        adam4(p, m, v, g, a, alpha);
        store4(prow, k, a.p_etype, p);
        if constexpr (MF32) {
            *reinterpret_cast<float4*>(mrow + (size_t)k * 4) = m;
            *reinterpret_cast<float4*>(vrow + (size_t)k * 4) = v;
        } else {
            store4(mrow, k, a.m_etype, m);
            store4(vrow, k, a.m_etype, v);
        }
    }
}

template <bool MF32>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(8, 8))) void k_adam_rows(AdamArgs a0, AdamArgs a1) {
    adam_rows_body<MF32, false>(a0, a1);
}
template <bool MF32>  // with the ComplEx / RotatE transforms of the contributions compiled in
__global__ __launch_bounds__(256) void k_adam_rows_xf(AdamArgs a0, AdamArgs a1) {
    adam_rows_body<MF32, true>(a0, a1);
}

// One launch for both tables without a first-level reduction before it.
//   blocks [0, NS0 * max_hot0), [.., + NS1 * max_hot1): hot rows, one workgroup per (row, 32 columns).
//     Lane = (slot, column group): eight contributions per load instruction (128 bytes of each),
//     sixteen such loads in flight; a lane adds its slot's contributions in sorted order, the
//     eight slots meet by butterfly shuffles (both operand orders give the same float), the four
//     waves' sums in LDS in wave order; eight lanes of wave 0 then update the 32 columns.
//   the remaining blocks: every other row, one wave per row, as k_adam_rows.
// columns per hot-row workgroup: 32 (128 bytes of every contribution per load; 16 and 8 columns
// measured slower: the same rows are then fetched by two and four times as many workgroups)
constexpr int kHotColumns = 32;
// loads in flight per lane: 8, and the kernel compiled for eight waves per SIMD (56 registers): the
// ordinary rows, one wave each, are bound by resident waves over the length of a wave's chain of
// dependent loads (22.8M-row workload 38.9 -> 33.8 us, 91.2M-row 32.2 -> 26.3 us against 16 loads
// and five waves; 4 and 16 loads at eight waves measured the same within a microsecond);
// four waves per workgroup (2, 8 and 16 measured slower)
constexpr int kHotLoads = 8, kHotWaves = 4;
// BYCHUNK: one hot workgroup per chunk of the plan instead of one per (row with chunks, 32
// columns).  A row of nch chunks has nch consecutive chunk workgroups; the first 1, 2, 4 or 8
// of them (the largest power of two <= min(nch, 8)) split its columns evenly and each sums all
// of the row's contributions over its share, the others return.  Rows with one chunk
// (17 .. 64 contributions) then cost one workgroup instead of eight.
template <bool MF32, bool BYCHUNK>
__global__ __launch_bounds__(kHotWaves * 64) __attribute__((amdgpu_waves_per_eu(8, 8))) void k_adam_rows_hot(AdamArgs a0, HotRows h0, AdamArgs a1, HotRows h1) {
    __shared__ __attribute__((aligned(16))) float part[kHotWaves - 1][BYCHUNK ? 256 : kHotColumns];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ns0 = (a0.Dp + kHotColumns - 1) / kHotColumns, ns1 = (a1.Dp + kHotColumns - 1) / kHotColumns;
    const int hot0 = BYCHUNK ? (a0.max_rows ? h0.n_chunks : 0) : ns0 * h0.max_hot;
    const int hot1 = BYCHUNK ? (a1.max_rows ? h1.n_chunks : 0) : ns1 * h1.max_hot;
    int b = blockIdx.x;
    if (b < hot0 + hot1) {
        const bool second = b >= hot0;
        const AdamArgs& a = second ? a1 : a0;
        const HotRows& h = second ? h1 : h0;
        if (second) b -= hot0;
        const int Dp = a.Dp;
        int u, col0, ncg;  // the row, this workgroup's first column and its groups of four columns
        if constexpr (BYCHUNK) {
            if (b >= (int)a.counts[1]) return;
            u = (int)h.chunk_row[b];
            const int q0 = (int)a.chunk_off[u], nch = (int)a.chunk_off[u + 1] - q0;
            const int shares = nch >= 8 ? 8 : nch >= 4 ? 4 : nch >= 2 ? 2 : 1;
            const int cb = b - q0;
            if (cb >= shares) return;
            const int HC = Dp / shares;
            col0 = cb * HC; ncg = HC / 4;
        } else {
            const int ns = second ? ns1 : ns0, hb = b / ns, cb = b - hb * ns;
            if (hb >= (int)h.hot_count[0]) return;
            u = (int)h.hot_rows[hb];
            col0 = cb * kHotColumns; ncg = kHotColumns / 4;
        }
        const int HS = 64 / ncg;  // contributions per load instruction (slots of a wave)
        const uint32_t key = a.uniq_key[u], pos = a.seg_start[u], n = a.seg_real[u];
        const float alpha = a.alpha[a.rows_per_alpha ? key / a.rows_per_alpha : 0u];
        const int cg = lane & (ncg - 1), slot = lane / ncg, col = col0 + cg * 4;
        const bool active = col < Dp;
        // this wave's quarter of the contributions, in whole groups of HS
        const uint32_t groups = (n + HS - 1) / HS, gshare = (groups + kHotWaves - 1) / kHotWaves;
        const uint32_t w0 = min(n, wave * gshare * HS), w1 = min(n, w0 + gshare * HS);
        const uint32_t* __restrict__ items = a.src.sorted_item + pos;
        const float* __restrict__ grad = a.src.grad;
        float4 acc = make_float4(0, 0, 0, 0);
        for (uint32_t j = w0; j < w1; j += kHotLoads * HS) {
            uint32_t c[kHotLoads];
            float4 v[kHotLoads];
#pragma unroll
            for (int x = 0; x < kHotLoads; ++x) {
                const uint32_t idx = j + x * HS + slot;
                c[x] = idx < w1 ? items[idx] : 0xffffffffu;
            }
#pragma unroll
            for (int x = 0; x < kHotLoads; ++x)
                v[x] = (active && c[x] != 0xffffffffu) ? *reinterpret_cast<const float4*>(grad + (size_t)c[x] * Dp + col)
                                                      : make_float4(0, 0, 0, 0);
#pragma unroll
            for (int x = 0; x < kHotLoads; ++x) acc = f4add(acc, v[x]);
        }
        if constexpr (BYCHUNK) {
            for (int off = ncg; off < 64; off <<= 1) {
                acc.x += __shfl_xor(acc.x, off, 64); acc.y += __shfl_xor(acc.y, off, 64);
                acc.z += __shfl_xor(acc.z, off, 64); acc.w += __shfl_xor(acc.w, off, 64);
            }
        } else {
#pragma unroll
            for (int off = kHotColumns / 4; off < 64; off <<= 1) {
                acc.x += __shfl_xor(acc.x, off, 64); acc.y += __shfl_xor(acc.y, off, 64);
                acc.z += __shfl_xor(acc.z, off, 64); acc.w += __shfl_xor(acc.w, off, 64);
            }
        }
        if (wave > 0 && slot == 0) *reinterpret_cast<float4*>(&part[wave - 1][cg * 4]) = acc;
        __syncthreads();
        if (wave != 0 || slot != 0 || !active) return;
        float4 g = acc;
#pragma unroll
        for (int w = 0; w < kHotWaves - 1; ++w) g = f4add(g, *reinterpret_cast<const float4*>(&part[w][cg * 4]));
        char* prow = a.p_base + (int64_t)key * a.pitch;
        char* mrow = a.m_base + (int64_t)key * a.pitch;
        char* vrow = a.v_base + (int64_t)key * a.pitch;
        if (a.grad_out) {
            float4 go = g;
            if (a.grad_out_add) go = f4add(go, *reinterpret_cast<const float4*>(a.grad_out_add + (size_t)u * Dp + col));
            *reinterpret_cast<float4*>(a.grad_out + (size_t)u * Dp + col) = go;
        }
        if (a.no_update) return;
        if (a.grad_add) g = f4add(g, *reinterpret_cast<const float4*>(a.grad_add + (size_t)u * Dp + col));
        float4 p = load4(prow, col, a.p_etype);
        float4 m = load4(mrow, col, a.m_etype), v = load4(vrow, col, a.m_etype);
        adam4(p, m, v, g, a, alpha);
        store4(prow, col, a.p_etype, p);
        store4(mrow, col, a.m_etype, m);
        store4(vrow, col, a.m_etype, v);
        return;
    }
    b -= hot0 + hot1;
    const int slabs = (max(a0.Dp, a1.Dp) + 255) / 256;   // a wave takes one slab of 256 columns of one row
    const int blocks0 = (a0.max_rows * slabs + kHotWaves - 1) / kHotWaves;
    const bool second = b >= blocks0;
    const AdamArgs& a = second ? a1 : a0;
    const int g = (second ? b - blocks0 : b) * kHotWaves + wave;
    const int u = g / slabs, slab = g - u * slabs;
    const int uc = min(u, a.max_rows - 1);
    const uint32_t key = a.uniq_key[uc];
    const uint32_t q0 = a.chunk_off[uc], q1 = a.chunk_off[uc + 1];
    const uint32_t pos = a.seg_start[uc], n_real = a.seg_real[uc];
    if (u >= (int)a.counts[0] || q1 > q0) return;  // a row with chunks belongs to the hot blocks
    const float alpha = a.alpha[a.rows_per_alpha ? key / a.rows_per_alpha : 0u];
    const int Dp = a.Dp;
    char* prow = a.p_base + (int64_t)key * a.pitch;
    char* mrow = a.m_base + (int64_t)key * a.pitch;
    char* vrow = a.v_base + (int64_t)key * a.pitch;
    {
        const int k = slab * 256 + lane * 4;
        const bool active = k < Dp;
        float4 g = make_float4(0, 0, 0, 0);
        if (n_real)  // wave-uniform: all lanes take part in the shuffles
            g = sum_contribs<4, false>(a.src, pos, n_real, k, Dp, lane, active);
        if (!active) return;
        float4 p = load4(prow, k, a.p_etype);
        float4 m, v;
        if constexpr (MF32) {
            m = *reinterpret_cast<const float4*>(mrow + (size_t)k * 4);
            v = *reinterpret_cast<const float4*>(vrow + (size_t)k * 4);
        } else {
            m = load4(mrow, k, a.m_etype);
            v = load4(vrow, k, a.m_etype);
        }
        if (a.grad_out) {
            float4 go = g;
            if (a.grad_out_add) go = f4add(go, *reinterpret_cast<const float4*>(a.grad_out_add + (size_t)u * Dp + k));
            *reinterpret_cast<float4*>(a.grad_out + (size_t)u * Dp + k) = go;
        }
        if (a.no_update) return;
        if (a.grad_add) g = f4add(g, *reinterpret_cast<const float4*>(a.grad_add + (size_t)u * Dp + k));
        adam4(p, m, v, g, a, alpha);
        store4(prow, k, a.p_etype, p);
        if constexpr (MF32) {
            *reinterpret_cast<float4*>(mrow + (size_t)k * 4) = m;
            *reinterpret_cast<float4*>(vrow + (size_t)k * 4) = v;
        } else {
            store4(mrow, k, a.m_etype, m);
            store4(vrow, k, a.m_etype, v);
        }
    }
}

// the per-chunk form takes row widths that split evenly into 1 .. 8 shares of whole 16-byte groups
static bool hot_by_chunk_ok(const AdamArgs& a, const HotRows& h) {
    return a.max_rows == 0 || (h.chunk_row && a.Dp >= 32 && a.Dp <= 256 && (a.Dp & (a.Dp - 1)) == 0);
}

void launch_adam_rows_hot2(const AdamArgs& a0, const HotRows& h0, const AdamArgs& a1, const HotRows& h1,
                           hipStream_t stream) {
    const bool by_chunk = hot_by_chunk_ok(a0, h0) && hot_by_chunk_ok(a1, h1);
    const int hot = by_chunk ? (a0.max_rows ? h0.n_chunks : 0) + (a1.max_rows ? h1.n_chunks : 0)
                             : ((a0.Dp + kHotColumns - 1) / kHotColumns) * h0.max_hot +
                               ((a1.Dp + kHotColumns - 1) / kHotColumns) * h1.max_hot;
    const int slabs = (std::max(a0.Dp, a1.Dp) + 255) / 256;
    const dim3 grid(hot + (a0.max_rows * slabs + kHotWaves - 1) / kHotWaves + (a1.max_rows * slabs + kHotWaves - 1) / kHotWaves);
    if (grid.x == 0) return;
    const bool f32 = (a0.max_rows == 0 || a0.m_etype == ET_F32) && (a1.max_rows == 0 || a1.m_etype == ET_F32);
    if (by_chunk && f32) hipLaunchKernelGGL((k_adam_rows_hot<true, true>), grid, dim3(kHotWaves * 64), 0, stream, a0, h0, a1, h1);
    else if (by_chunk) hipLaunchKernelGGL((k_adam_rows_hot<false, true>), grid, dim3(kHotWaves * 64), 0, stream, a0, h0, a1, h1);
    else if (f32) hipLaunchKernelGGL((k_adam_rows_hot<true, false>), grid, dim3(kHotWaves * 64), 0, stream, a0, h0, a1, h1);
    else hipLaunchKernelGGL((k_adam_rows_hot<false, false>), grid, dim3(kHotWaves * 64), 0, stream, a0, h0, a1, h1);
}

static void launch_adam_kernel(const AdamArgs& a0, const AdamArgs& a1, hipStream_t stream) {
    const int slabs = (std::max(a0.Dp, a1.Dp) + 255) / 256;
    const dim3 grid((a0.max_rows * slabs + 3) / 4 + (a1.max_rows * slabs + 3) / 4);
    if (grid.x == 0) return;
    const bool f32 = (a0.max_rows == 0 || a0.m_etype == ET_F32) && (a1.max_rows == 0 || a1.m_etype == ET_F32);
    const bool xf = (a0.max_rows && a0.src.transform >= 3) || (a1.max_rows && a1.src.transform >= 3);
    if (f32 && !xf) hipLaunchKernelGGL((k_adam_rows<true>), grid, dim3(256), 0, stream, a0, a1);
    else if (f32) hipLaunchKernelGGL((k_adam_rows_xf<true>), grid, dim3(256), 0, stream, a0, a1);
    else if (!xf) hipLaunchKernelGGL((k_adam_rows<false>), grid, dim3(256), 0, stream, a0, a1);
    else hipLaunchKernelGGL((k_adam_rows_xf<false>), grid, dim3(256), 0, stream, a0, a1);
}
void launch_adam_rows(const AdamArgs& a, hipStream_t stream) {
    AdamArgs none = a;
    none.max_rows = 0;
    launch_adam_kernel(a, none, stream);
}
void launch_adam_rows2(const AdamArgs& a0, const AdamArgs& a1, hipStream_t stream) {
    launch_adam_kernel(a0, a1, stream);
}

// One workgroup per shard; a fixed order of additions whatever the launch: thread t takes entries
// t, t + 256, ... of the shard's (step, part) pairs, lanes meet by butterfly, waves in wave order.
__global__ __launch_bounds__(256) void k_loss_finalize(const float* __restrict__ loss_part, int n_step,
                                                       int S, int n_part, float scale,
                                                       float* __restrict__ loss,
                                                       const float* __restrict__ extra) {
    __shared__ float red[4];
    const int s = blockIdx.x, tid = threadIdx.x;
    const int n = n_step * n_part;
    float acc = 0.f;
    for (int e = tid; e < n; e += 256) {
        const int i = e / n_part, t = e - i * n_part;
        acc += loss_part[((size_t)i * S + s) * n_part + t];
    }
    if (extra)
        for (int i = tid; i < n_step; i += 256) acc += extra[(size_t)i * S + s];
    acc = wave_sum(acc);
    if ((tid & 63) == 0) red[tid >> 6] = acc;
    __syncthreads();
    if (tid == 0) loss[s] = (red[0] + red[1] + red[2] + red[3]) * scale;
}

// One workgroup per (step, shard): the sum of that step's parts, in the same fixed order.
__global__ __launch_bounds__(256) void k_loss_step_sums(const float* __restrict__ loss_part, int n_part,
                                                        float* __restrict__ step_sums) {
    __shared__ float red[4];
    const float* part = loss_part + (size_t)blockIdx.x * n_part;
    const int tid = threadIdx.x;
    float acc = 0.f;
    for (int t = tid; t < n_part; t += 256) acc += part[t];
    acc = wave_sum(acc);
    if ((tid & 63) == 0) red[tid >> 6] = acc;
    __syncthreads();
    if (tid == 0) step_sums[blockIdx.x] = red[0] + red[1] + red[2] + red[3];
}

// `step_sums` (n_step * S floats, may be null): scratch for the two-level sum that long part lists take.
void launch_loss_finalize(const float* loss_part, int n_step, int S, int n_part, float scale,
                          float* loss, hipStream_t stream, const float* extra, float* step_sums) {
    if (step_sums && n_part > 256 && n_step > 1) {
        hipLaunchKernelGGL(k_loss_step_sums, dim3(n_step * S), dim3(256), 0, stream, loss_part, n_part, step_sums);
        loss_part = step_sums;
        n_part = 1;
    }
    hipLaunchKernelGGL(k_loss_finalize, dim3(S), dim3(256), 0, stream, loss_part, n_step, S, n_part,
                       scale, loss, extra);
}

// --------------------------------------------------------------------------
// norm regularisers: one wave per distinct row, two passes over the row (sums, then gradients)

// |x^p| and its share of the gradient |x^p| / x (0 at x = 0: the reference's pow backward
// divides by x + (x == 0), src/pag/pag.cpp:483-503)
DEVINL float abs_pow(float x, float p) { return fabsf(powf(x, p)); }

__global__ __launch_bounds__(256) void k_reg_rows(RegArgs a) {
    const int lane = threadIdx.x & 63;
    const int u = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= (int)a.counts[0]) return;
    const uint32_t key = a.uniq_key[u];
    const float mult = (float)((a.seg_start[u + 1] - a.seg_start[u]) - a.seg_real[u]);
    const char* erow = a.emb_base + (int64_t)key * a.pitch;
    const float* hrow = a.hidden ? a.hidden + (size_t)u * a.Dp : nullptr;
    float sum[3] = {0.f, 0.f, 0.f};
    for (int k = lane; k < a.D; k += 64) {
        const float v = load1(erow, k, a.emb_etype), h = hrow ? hrow[k] : v;
        if (a.weight[0] > 0.f) sum[0] += abs_pow(v, a.power[0]);
        if (a.weight[1] > 0.f) sum[1] += abs_pow(h - v, a.power[1]);
        if (a.weight[2] > 0.f) sum[2] += abs_pow(h, a.power[2]);
    }
    float norm[3], coef[3], loss = 0.f;
#pragma unroll
    for (int q = 0; q < 3; ++q) {
        sum[q] = wave_sum(sum[q]);
        norm[q] = a.weight[q] > 0.f ? powf(sum[q], 1.f / a.power[q]) : 0.f;
        // d loss / d x_k = seed * (norm / sum) * |x_k^p| / x_k, seed = uses * mult * weight * loss_scale
        coef[q] = sum[q] != 0.f ? a.uses * mult * a.weight[q] * a.loss_scale * norm[q] / sum[q] : 0.f;
        loss += a.uses * mult * a.weight[q] * norm[q];
    }
    if (lane == 0) a.loss_row[u] = a.accumulate ? a.loss_row[u] + loss : loss;
    for (int k = lane; k < a.Dp; k += 64) {
        float gv = 0.f, gf = 0.f;
        if (k < a.D) {
            const float v = load1(erow, k, a.emb_etype), h = hrow ? hrow[k] : v, f = h - v;
            if (a.weight[0] > 0.f && v != 0.f) gv += coef[0] * abs_pow(v, a.power[0]) / v;
            if (a.weight[1] > 0.f && f != 0.f) gf += coef[1] * abs_pow(f, a.power[1]) / f;
            if (a.weight[2] > 0.f && h != 0.f) {
                const float gh = coef[2] * abs_pow(h, a.power[2]) / h;
                gv += gh; gf += gh;
            }
        }
        a.add_val[(size_t)u * a.Dp + k] = a.accumulate ? a.add_val[(size_t)u * a.Dp + k] + gv : gv;
        if (a.add_fh) a.add_fh[(size_t)u * a.Dp + k] = gf;
    }
}
void launch_reg_rows(const RegArgs& a, hipStream_t stream) {
    hipLaunchKernelGGL(k_reg_rows, dim3((a.max_rows + 3) / 4), dim3(256), 0, stream, a);
}

__global__ __launch_bounds__(64) void k_reg_loss(const uint32_t* __restrict__ uniq_key,
                                                 const uint32_t* __restrict__ counts,
                                                 const float* __restrict__ loss_row, uint32_t rows_per_shard,
                                                 float* __restrict__ out) {
    const int s = blockIdx.x, lane = threadIdx.x;
    const int U = (int)counts[0];
    float part = 0.f;
    for (int u = lane; u < U; u += 64)
        if (uniq_key[u] / rows_per_shard == (uint32_t)s) part += loss_row[u];
    part = wave_sum(part);
    if (lane == 0) out[s] = part;
}
void launch_reg_loss(const uint32_t* uniq_key, const uint32_t* counts, const float* loss_row,
                     uint32_t rows_per_shard, int S, float* out, hipStream_t stream) {
    hipLaunchKernelGGL(k_reg_loss, dim3(S), dim3(64), 0, stream, uniq_key, counts, loss_row, rows_per_shard, out);
}

// --------------------------------------------------------------------------
// feature projection (src/poplar_kge.cpp:451-462): one wave per distinct row

__global__ __launch_bounds__(256) void k_hidden_fwd(FeatureArgs a, float* __restrict__ hidden) {
    const int lane = threadIdx.x & 63;
    const int u = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= (int)a.counts[0]) return;
    const uint32_t key = a.uniq_key[u];
    const char* erow = a.emb_base + (int64_t)key * a.pitch;
    const char* frow = a.feat_base + (int64_t)key * a.pitch;
    for (int k = lane * 4; k < a.Dp; k += 256) {
        float4 h = a.emb_base ? load4(erow, k, a.emb_etype) : make_float4(0, 0, 0, 0);
        for (int f = 0; f < a.Fp; f += 4) {
            float4 x = load4(frow, f, a.feat_etype);
            if (a.round_bf16) x = round4_bf16(x);
            const float xv[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float4 w = *reinterpret_cast<const float4*>(a.proj + (size_t)(f + i) * a.Dp + k);
                if (a.round_bf16) w = round4_bf16(w);
                h.x = fmaf(xv[i], w.x, h.x); h.y = fmaf(xv[i], w.y, h.y);
                h.z = fmaf(xv[i], w.z, h.z); h.w = fmaf(xv[i], w.w, h.w);
            }
        }
        *reinterpret_cast<float4*>(hidden + (size_t)u * a.Dp + k) = h;
    }
}

// The distinct rows' features as dense float32 [max_rows, Fp], rows past the
// count zero: the operand both feature products read.  One wave per row.
__global__ __launch_bounds__(256) void k_gather_features(FeatureArgs a, float* __restrict__ featd,
                                                         uint16_t* __restrict__ feat16) {
    const int lane = threadIdx.x & 63;
    const int u = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= a.max_rows) return;
    const bool live = u < (int)a.counts[0];
    const char* frow = a.feat_base + (int64_t)(live ? a.uniq_key[u] : 0u) * a.pitch;
    for (int f = lane * 4; f < a.Fp; f += 256) {
        const float4 x = live ? load4(frow, f, a.feat_etype) : make_float4(0, 0, 0, 0);
        if (feat16) {
            uint2 raw;
            raw.x = (uint32_t)f32_to_bf16(x.x) | ((uint32_t)f32_to_bf16(x.y) << 16);
            raw.y = (uint32_t)f32_to_bf16(x.z) | ((uint32_t)f32_to_bf16(x.w) << 16);
            *reinterpret_cast<uint2*>(feat16 + (size_t)u * a.Fp + f) = raw;
        } else {
            *reinterpret_cast<float4*>(featd + (size_t)u * a.Fp + f) = a.round_bf16 ? round4_bf16(x) : x;
        }
    }
}

// out = in rounded to bfloat16 (kept as float32); n % 4 == 0
__global__ __launch_bounds__(256) void k_round_bf16_copy(const float* __restrict__ in, int64_t n,
                                                         float* __restrict__ out) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i < n) *reinterpret_cast<float4*>(out + i) = round4_bf16(*reinterpret_cast<const float4*>(in + i));
}

// bfloat16 feature products (with bfloat16 scoring): both are C = A . Bt^T products
static bool feature_bf16_ok(const FeatureArgs& a) {
    return a.use_mfma && a.feat16 && gemm_nt_bf16_ok(a.max_rows, a.Dp, a.Fp) &&
           gemm_nt_bf16_ok(a.Fp, a.Dp, a.max_rows);
}

static bool feature_mfma_ok(const FeatureArgs& a) {
    return a.use_mfma && a.featd && (a.Dp & 3) == 0 && (a.Fp & 3) == 0;
}

static RowSource dense_rows(const float* base, int cols) {
    RowSource r;
    r.base = reinterpret_cast<const char*>(base); r.pitch = (int64_t)cols * 4; r.etype = ET_F32;
    r.index = nullptr; r.count = cols; r.vec = 1;
    return r;
}

// hidden[u, :] = embedding[key u, :] + feature[u, :] . W as a [U x Fp] . [Fp x Dp]
// product on the matrix cores (the scoring backward's dot kernel: coefficient
// matrix = dense features, other rows = W), the embedding added in its epilogue.
void launch_hidden_fwd(const FeatureArgs& a, float* hidden, hipStream_t stream) {
    if (feature_bf16_ok(a)) {
        // hidden [U, Dp] = features [U, Fp] . W [Fp, Dp] + embedding: A = features, Bt = W^T
        hipLaunchKernelGGL(k_gather_features, dim3((a.max_rows + 3) / 4), dim3(256), 0, stream, a,
                           (float*)nullptr, a.feat16);
        GemmNT g = {};
        g.A = a.feat16; g.lda = a.Fp; g.C = hidden; g.ldc = a.Dp;
        g.Bt = reinterpret_cast<const uint16_t*>(a.proj); g.ldb = a.Dp; g.b_kmajor = 2;  // W [Fp, Dp] float32 as it lies
        g.M = a.max_rows; g.N = a.Dp; g.K = a.Fp; g.batches = 1;
        g.add_base = a.emb_base; g.add_pitch = a.pitch; g.add_etype = a.emb_etype;
        g.add_index = a.uniq_key; g.add_count = a.counts;
        g.m_limit = a.counts;  // rows past the distinct count are never read
        launch_gemm_nt_bf16(g, stream);
        return;
    }
    if (!feature_mfma_ok(a)) {
        hipLaunchKernelGGL(k_hidden_fwd, dim3((a.max_rows + 3) / 4), dim3(256), 0, stream, a, hidden);
        return;
    }
    hipLaunchKernelGGL(k_gather_features, dim3((a.max_rows + 3) / 4), dim3(256), 0, stream, a, a.featd,
                       (uint16_t*)nullptr);
    const float* w = a.proj;
    if (a.round_bf16) {  // bfloat16 operands at shapes the bfloat16 product does not take
        const int64_t n = (int64_t)a.Fp * a.Dp;
        hipLaunchKernelGGL(k_round_bf16_copy, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, stream,
                           a.proj, n, a.projR);
        w = a.projR;
    }
    BwdParams p = {};
    p.ent_a = p.ent_b = dense_rows(w, a.Dp);
    p.coef = a.featd; p.grad = hidden;
    p.S = 1; p.B = a.max_rows; p.T = a.Fp; p.Dp = a.Dp;
    p.side_b = 0; p.vec_out = 1; p.use_mfma = 1;
    p.add_base = a.emb_base; p.add_pitch = a.pitch; p.add_etype = a.emb_etype;
    p.add_index = a.uniq_key; p.add_count = a.counts;
    launch_bwd(p, DIST_DOT, stream);
}

// gproj[f, k] = sum_u feature[u, f] * grad_rows[u, k]; block = 4 feature rows x 64 float4 columns
__global__ __launch_bounds__(256) void k_proj_grad(FeatureArgs a, const float* __restrict__ grad_rows,
                                                   float* __restrict__ gproj) {
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int k = (blockIdx.x * 64 + lane) * 4;
    if (f >= a.Fp || k >= a.Dp) return;
    const int U = a.counts[0];
    float4 acc = make_float4(0, 0, 0, 0);
    for (int u = 0; u < U; ++u) {
        const char* frow = a.feat_base + (int64_t)a.uniq_key[u] * a.pitch;
        float x;
        if (a.feat_etype == ET_F32) x = reinterpret_cast<const float*>(frow)[f];
        else if (a.feat_etype == ET_F16) x = __half2float(reinterpret_cast<const __half*>(frow)[f]);
        else x = bf16_to_f32(reinterpret_cast<const uint16_t*>(frow)[f]);
        if (a.round_bf16) x = bf16_to_f32(f32_to_bf16(x));
        const float4 g = *reinterpret_cast<const float4*>(grad_rows + (size_t)u * a.Dp + k);
        acc.x = fmaf(x, g.x, acc.x); acc.y = fmaf(x, g.y, acc.y);
        acc.z = fmaf(x, g.z, acc.z); acc.w = fmaf(x, g.w, acc.w);
    }
    *reinterpret_cast<float4*>(gproj + (size_t)f * a.Dp + k) = acc;
}

// out[i] = sum over the `ns` partial arrays of part[s][i], in order (n % 4 == 0)
__global__ __launch_bounds__(256) void k_sum_splits(const float* __restrict__ part, int ns, int64_t n,
                                                    float* __restrict__ out) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    float4 acc = *reinterpret_cast<const float4*>(part + i);
    for (int s = 1; s < ns; ++s) acc = f4add(acc, *reinterpret_cast<const float4*>(part + (size_t)s * n + i));
    *reinterpret_cast<float4*>(out + i) = acc;
}

void launch_proj_grad(const FeatureArgs& a, const float* grad_rows, float* gproj,
                      hipStream_t stream) {
    if (feature_bf16_ok(a)) {
        // gproj [Fp, Dp] = features^T [Fp, U] . grad_rows [U, Dp]: both operands read as they lie,
        // with the contraction index outermost (the float32 gradient rows rounded while staged);
        // rows past the distinct count are zero in the features and finite in grad_rows
        // (the contraction stops at the distinct count, rounded up to a slab)
        GemmNT g = {};
        g.A = a.feat16; g.lda = a.Fp; g.a_kmajor = 1;  // the features as they lie, [U, Fp]
        g.Bt = reinterpret_cast<const uint16_t*>(grad_rows); g.ldb = a.Dp; g.b_kmajor = 2;  // [U, Dp] float32 as they lie
        g.C = gproj; g.ldc = a.Dp;
        g.M = a.Fp; g.N = a.Dp; g.K = a.max_rows; g.batches = 1;
        g.part = a.gproj_part;  // [16, Fp, Dp]: room for every split
        g.k_limit = a.counts;
        launch_gemm_nt_bf16(g, stream);
        return;
    }
    if (feature_mfma_ok(a)) {
        // gproj = features^T . grad_rows, [Fp x U] . [U x Dp]: the dot kernel's tail side
        // (coefficient rows run along the contraction).  Rows past the distinct count
        // are zero in the dense features and finite in grad_rows, so they add nothing.
        // The output has few tiles, so the contraction is split over `ns` blocks of
        // rows whose partial products are then added in block order.
        int ns = 1;
        while (ns < 16 && a.max_rows % (2 * ns * 32) == 0 && a.gproj_part) ns *= 2;
        BwdParams p = {};
        p.ent_a = p.ent_b = dense_rows(grad_rows, a.Dp);
        p.coef = a.featd; p.grad = ns > 1 ? a.gproj_part : gproj;
        p.S = ns; p.B = a.max_rows / ns; p.T = a.Fp; p.Dp = a.Dp;
        p.side_b = 1; p.vec_out = 1; p.use_mfma = 1;
        launch_bwd(p, DIST_DOT, stream);
        if (ns > 1) {
            const int64_t n = (int64_t)a.Fp * a.Dp;
            hipLaunchKernelGGL(k_sum_splits, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, stream,
                               a.gproj_part, ns, n, gproj);
        }
        return;
    }
    dim3 grid((a.Dp / 4 + 63) / 64, (a.Fp + 3) / 4);
    hipLaunchKernelGGL(k_proj_grad, grid, dim3(256), 0, stream, a, grad_rows, gproj);
}

// --------------------------------------------------------------------------
// table access

// One wave per row, 16 bytes per lane per iteration when the row allows it.
__global__ __launch_bounds__(256) void k_rows_copy(const char* __restrict__ src,
                                                   char* __restrict__ dst,
                                                   const uint32_t* __restrict__ idx, int64_t n,
                                                   int64_t row_bytes, int scatter, int vec16) {
    const int lane = threadIdx.x & 63;
    const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (i >= n) return;
    const int64_t r = idx[i];
    const char* s = scatter ? src + i * row_bytes : src + r * row_bytes;
    char* d = scatter ? dst + r * row_bytes : dst + i * row_bytes;
    if (vec16) {
        for (int64_t b = (int64_t)lane * 16; b < row_bytes; b += 64 * 16)
            *reinterpret_cast<uint4*>(d + b) = *reinterpret_cast<const uint4*>(s + b);
    } else {
        for (int64_t b = (int64_t)lane * 4; b < row_bytes; b += 64 * 4)
            *reinterpret_cast<uint32_t*>(d + b) = *reinterpret_cast<const uint32_t*>(s + b);
    }
}

void launch_rows_gather(const void* buf, const uint32_t* idx, void* out, int64_t n,
                        int64_t row_bytes, hipStream_t stream) {
    if (n == 0) return;
    const int vec16 = (row_bytes % 16 == 0) && ((uintptr_t)buf % 16 == 0) && ((uintptr_t)out % 16 == 0);
    hipLaunchKernelGGL(k_rows_copy, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, stream,
                       (const char*)buf, (char*)out, idx, n, row_bytes, 0, vec16);
}

void launch_rows_scatter(void* buf, const uint32_t* idx, const void* data, int64_t n,
                         int64_t row_bytes, hipStream_t stream) {
    if (n == 0) return;
    const int vec16 = (row_bytes % 16 == 0) && ((uintptr_t)buf % 16 == 0) && ((uintptr_t)data % 16 == 0);
    hipLaunchKernelGGL(k_rows_copy, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, stream,
                       (const char*)data, (char*)buf, idx, n, row_bytes, 1, vec16);
}

DEVINL void store1(char* sec, int k, int etype, float v) {
    if (etype == ET_F32) reinterpret_cast<float*>(sec)[k] = v;
    else if (etype == ET_BF16) reinterpret_cast<uint16_t*>(sec)[k] = f32_to_bf16(v);
    else reinterpret_cast<__half*>(sec)[k] = __float2half_rn(v);
}

// logical column c of [emb D | m D | sqrt v D | feature F] -> (section byte offset, index, type)
DEVINL void locate(const RowLayout& L, int c, int64_t& off, int& k, int& et) {
    if (c < L.D) { off = 0; k = c; et = L.emb_etype; }
    else if (c < 2 * L.D) { off = L.off_m; k = c - L.D; et = L.mom_etype; }
    else if (c < 3 * L.D) { off = L.off_s; k = c - 2 * L.D; et = L.mom_etype; }
    else { off = L.off_f; k = c - 3 * L.D; et = L.feat_etype; }
}

__global__ __launch_bounds__(256) void k_rows_to_logical(RowLayout L, const char* __restrict__ base,
                                                         const uint64_t* __restrict__ rows, int64_t n,
                                                         float* __restrict__ out) {
    const int W = 3 * L.D + L.F;
    const int64_t i = blockIdx.x;
    if (i >= n) return;
    const char* row = base + (int64_t)rows[i] * L.pitch;
    for (int c = threadIdx.x; c < W; c += 256) {
        int64_t off; int k, et;
        locate(L, c, off, k, et);
        out[i * W + c] = load1(row + off, k, et);
    }
}

__global__ __launch_bounds__(256) void k_rows_from_logical(RowLayout L, char* __restrict__ base,
                                                           const uint64_t* __restrict__ rows,
                                                           int64_t n, const float* __restrict__ in) {
    const int W = 3 * L.D + L.F;
    const int64_t i = blockIdx.x;
    if (i >= n) return;
    char* row = base + (int64_t)rows[i] * L.pitch;
    for (int c = threadIdx.x; c < W; c += 256) {
        int64_t off; int k, et;
        locate(L, c, off, k, et);
        store1(row + off, k, et, in[i * W + c]);
    }
}

void launch_rows_to_logical(const RowLayout& L, const char* base, const uint64_t* rows, int64_t n,
                            float* out, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(k_rows_to_logical, dim3((unsigned)n), dim3(256), 0, stream, L, base, rows, n, out);
}
void launch_rows_from_logical(const RowLayout& L, char* base, const uint64_t* rows, int64_t n,
                              const float* in, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(k_rows_from_logical, dim3((unsigned)n), dim3(256), 0, stream, L, base, rows, n, in);
}

// counter-based normal generator: two rounds of a 64-bit mix, then Box-Muller
DEVINL uint64_t mix64(uint64_t x) {
    x ^= x >> 30; x *= 0xbf58476d1ce4e5b9ull;
    x ^= x >> 27; x *= 0x94d049bb133111ebull;
    x ^= x >> 31;
    return x;
}
DEVINL float normal_at(uint32_t seed, uint64_t row, uint32_t col) {
    const uint64_t h = mix64(mix64(((uint64_t)seed << 32) ^ row * 0x9e3779b97f4a7c15ull) + col);
    const float u1 = ((uint32_t)(h >> 40) + 1u) * (1.0f / 16777217.0f);  // (0, 1)
    const float u2 = (uint32_t)(h & 0xffffffu) * (1.0f / 16777216.0f);   // [0, 1)
    return sqrtf(-2.f * logf(u1)) * cospif(2.f * u2);
}

// Model::writeEntity (src/poplar_kge.cpp:864-871): emb ~ N(0, sigma), zero
// moments, host features; padding columns are zero.
__global__ __launch_bounds__(256) void k_init_rows(RowLayout L, char* __restrict__ base,
                                                   const uint64_t* __restrict__ rows, int64_t n,
                                                   const float* __restrict__ features, float sigma,
                                                   uint32_t seed) {
    const int64_t i = blockIdx.x;
    if (i >= n) return;
    const uint64_t r = rows[i];
    char* row = base + (int64_t)r * L.pitch;
    for (int k = threadIdx.x; k < L.Dp; k += 256) {
        store1(row, k, L.emb_etype, k < L.D ? sigma * normal_at(seed, r, k) : 0.f);
        store1(row + L.off_m, k, L.mom_etype, 0.f);
        store1(row + L.off_s, k, L.mom_etype, 0.f);
    }
    for (int f = threadIdx.x; f < L.Fp; f += 256)
        store1(row + L.off_f, f, L.feat_etype, f < L.F ? features[i * L.F + f] : 0.f);
}

void launch_init_rows(const RowLayout& L, char* base, const uint64_t* rows, int64_t n,
                      const float* features, float sigma, uint32_t seed, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(k_init_rows, dim3((unsigned)n), dim3(256), 0, stream, L, base, rows, n,
                       features, sigma, seed);
}

// --------------------------------------------------------------------------
// standalone ops

static RowSource plain_rows(const float* ptr, int D) {
    RowSource r;
    r.base = (const char*)ptr; r.pitch = (int64_t)D * 4; r.etype = ET_F32; r.index = nullptr;
    r.count = D; r.vec = (D % 4 == 0) && ((uintptr_t)ptr % 16 == 0);
    return r;
}

void launch_distance(int dist_fn, const float* a, const float* b, float* out, int M, int N, int D,
                     hipStream_t stream) {
    FwdParams p;
    p.sh.S = 1; p.sh.B = M; p.sh.T = N; p.sh.Dp = D;
    p.sh.score_fn = SCORE_TRANSE; p.sh.dist_fn = dist_fn; p.sh.loss_fn = LOSS_LOGSIGMOID;
    p.sh.gamma = 0.f; p.sh.loss_scale = 1.f; p.sh.softmax_correction = 0.f;
    p.sh.negative_adversarial_scale = 0.f;
    p.sh.use_mfma = 1; p.sh.operands_dense = 0;
    p.ent_a = plain_rows(a, D); p.ent_b = plain_rows(b, D);
    p.rel = nullptr; p.crel = nullptr; p.clabel = nullptr;
    p.coef = out; p.dist = nullptr; p.loss_part = nullptr;
    p.a_rel_mode = 0; p.out_mode = 2;
    p.a_c0 = 0; p.b_c0 = 0; p.nearflag = nullptr;
    launch_fwd(p, stream);
}

__global__ __launch_bounds__(256) void k_adam_flat(float* __restrict__ p, float* __restrict__ m,
                                                   float* __restrict__ v, const float* __restrict__ g,
                                                   int64_t n, AdamArgs a, float alpha) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float vi = v[i];
    if (a.v_is_sqrt) vi = vi * vi;
    const float mi = a.beta_m * m[i] + a.one_minus_beta_m * g[i];
    vi = a.beta_v * vi + a.one_minus_beta_v * g[i] * g[i];
    p[i] = p[i] - alpha * (mi / (sqrtf(vi) + a.epsilon) + a.weight_decay * p[i]);
    m[i] = mi;
    v[i] = a.v_is_sqrt ? sqrtf(vi) : vi;
}

void launch_adam_flat(float* p, float* m, float* v, const float* g, int64_t n, float alpha,
                      float beta_m, float beta_v, float epsilon, float weight_decay, int v_is_sqrt,
                      hipStream_t stream) {
    if (n == 0) return;
    AdamArgs a = {};
    a.beta_m = beta_m; a.beta_v = beta_v;
    a.one_minus_beta_m = 1.f - beta_m; a.one_minus_beta_v = 1.f - beta_v;
    a.epsilon = epsilon; a.weight_decay = weight_decay; a.v_is_sqrt = v_is_sqrt;
    hipLaunchKernelGGL(k_adam_flat, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p, m, v,
                       g, n, a, alpha);
}

__global__ __launch_bounds__(256) void k_fill_u32(uint32_t* p, uint32_t value, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = value;
}
void launch_fill_u32(uint32_t* p, uint32_t value, int64_t n, hipStream_t stream) {
    if (n == 0) return;
    hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p, value, n);
}

// out[r, :] = sum of the partial rows of table row r's chunks (second level
// of the segmented reduction without an optimiser step)
__global__ __launch_bounds__(256) void k_sum_partials_rows(const uint32_t* __restrict__ chunk_off,
                                                           const float* __restrict__ partial,
                                                           int64_t rows, int64_t cols,
                                                           float* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const uint32_t q0 = chunk_off[r], q1 = chunk_off[r + 1];
    if (cols & 3) {
        for (int64_t k = lane; k < cols; k += 64) {
            float g = 0.f;
            for (uint32_t q = q0; q < q1; ++q) g += partial[(size_t)q * cols + k];
            out[r * cols + k] = g;
        }
        return;
    }
    for (int64_t k = lane * 4; k < cols; k += 256) {
        float4 g = make_float4(0, 0, 0, 0);
        for (uint32_t q = q0; q < q1; ++q)
            g = f4add(g, *reinterpret_cast<const float4*>(partial + (size_t)q * cols + k));
        *reinterpret_cast<float4*>(out + r * cols + k) = g;
    }
}
void launch_sum_partials_rows(const uint32_t* chunk_off, const float* partial, int64_t rows,
                              int64_t cols, float* out, hipStream_t stream) {
    hipLaunchKernelGGL(k_sum_partials_rows, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream,
                       chunk_off, partial, rows, cols, out);
}

// --------------------------------------------------------------------------
// TransH (src/poplar_kge.cpp:539-565).  Per positive b: the unit normal n_b = w / |w| of its
// relation's hyperplane (w = the relation_normal row) and the predicted tail
// p_b = h - n (n . h) + r.  Score of (b, t): gamma - sum_k |e_btk| with
// e_btk = p_bk - (tau_tk - n_bk c_bt), c_bt = n_b . tau_t, whatever distance_fn says.
// Two dense float32 operand matrices [R, Dp]: `pt` rows [0, SB) predicted tails, rows
// [SB, R) tails; `nt` rows [0, SB) unit normals, rows [SB, R) the same tails, so that c and
// its backward (d n += dc tau, d tau += dc^T n) are the ordinary dot-product scoring
// kernels on `nt`.  The relation table holds the normals as rows [n_rel, 2 n_rel).

// heads of `pt` (holding the gathered head rows h) -> p; heads of `nt` -> n.  One wave per positive.
__global__ __launch_bounds__(256) void k_transh_predict(const float* __restrict__ rel,
                                                        const uint32_t* __restrict__ crel, int n_rel,
                                                        int n_head, int Dp, float* __restrict__ pt,
                                                        float* __restrict__ nt) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (c >= n_head) return;
    const uint32_t r = crel[c];
    const float* w = rel + (size_t)(n_rel + r) * Dp;
    const float* dr = rel + (size_t)r * Dp;
    float* h = pt + (size_t)c * Dp;
    float ss = 0.f;
    for (int k = lane * 4; k < Dp; k += 256) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + k);
        ss += w4.x * w4.x + w4.y * w4.y + w4.z * w4.z + w4.w * w4.w;
    }
    const float nrm = sqrtf(wave_sum(ss));
    float a = 0.f;
    for (int k = lane * 4; k < Dp; k += 256) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + k);
        const float4 h4 = *reinterpret_cast<const float4*>(h + k);
        a += (w4.x / nrm) * h4.x + (w4.y / nrm) * h4.y + (w4.z / nrm) * h4.z + (w4.w / nrm) * h4.w;
    }
    a = wave_sum(a);
    for (int k = lane * 4; k < Dp; k += 256) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + k);
        const float4 h4 = *reinterpret_cast<const float4*>(h + k);
        const float4 d4 = *reinterpret_cast<const float4*>(dr + k);
        const float4 n4 = make_float4(w4.x / nrm, w4.y / nrm, w4.z / nrm, w4.w / nrm);
        float4 p4 = make_float4((h4.x - n4.x * a) + d4.x, (h4.y - n4.y * a) + d4.y, (h4.z - n4.z * a) + d4.z,
                                (h4.w - n4.w * a) + d4.w);
        *reinterpret_cast<float4*>(h + k) = p4;
        *reinterpret_cast<float4*>(nt + (size_t)c * Dp + k) = n4;
    }
}
void launch_transh_predict(const float* rel, const uint32_t* crel, int n_rel, int n_head, int Dp, float* pt,
                           float* nt, hipStream_t stream) {
    hipLaunchKernelGGL(k_transh_predict, dim3((n_head + 3) / 4), dim3(256), 0, stream, rel, crel, n_rel, n_head,
                       Dp, pt, nt);
}

DEVINL float sign0(float t) { return (t > 0.f ? 1.f : 0.f) - (t < 0.f ? 1.f : 0.f); }

// Forward over 64 x 64 score tiles.  OM 0: fused logsigmoid loss, `coef` receives the
// coefficient G = d loss / d distance (scaled) and `dcm` G * q with q_bt = sum_k sign(e_btk) n_bk
// (= d loss / d c_bt); OM 1: `coef` receives the raw score and `dcm` q (the loss rows turn the
// scores into G, launch_mul_rows then forms G * q).
template <int OM>
__global__ __launch_bounds__(256) void k_transh_fwd(TranshFwd p) {
    __shared__ __attribute__((aligned(16))) float As[BK][LDP];
    __shared__ __attribute__((aligned(16))) float Ns[BK][LDP];
    __shared__ __attribute__((aligned(16))) float Bs[BK][LDP];
    __shared__ float red[4];
    __shared__ uint32_t label_s[kScoreTile];
    const ScoreShape& sh = p.sh;
    const TileId tile = xcd_tile((sh.T + kScoreTile - 1) / kScoreTile, (sh.B + kScoreTile - 1) / kScoreTile, sh.S);
    const int d = tile.z, m0 = tile.y * kScoreTile, n0 = tile.x * kScoreTile;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int B = sh.B, T = sh.T, Dp = sh.Dp;
    if (OM == 0 && tid < kScoreTile) label_s[tid] = m0 + tid < B ? p.clabel[d * B + m0 + tid] : 0u;
    const int lr = tid >> 3, k4 = (tid & 7) * 4;
    const int n_head = sh.S * B;

    float cm[4][4], acc[4][4], q[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            cm[i][j] = (m < B && n < T) ? p.cmat[((size_t)d * B + m) * T + n] : 0.f;
            acc[i][j] = 0.f;
            q[i][j] = 0.f;
        }

    for (int k0 = 0; k0 < Dp; k0 += BK) {
        const int k = k0 + k4;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int m = m0 + lr + 32 * h, n = n0 + lr + 32 * h;
            float4 a = make_float4(0, 0, 0, 0), nn = a, b = a;
            if (k < Dp) {
                if (m < B) {
                    a = *reinterpret_cast<const float4*>(p.pt + (size_t)(d * B + m) * Dp + k);
                    nn = *reinterpret_cast<const float4*>(p.nt + (size_t)(d * B + m) * Dp + k);
                }
                if (n < T) b = *reinterpret_cast<const float4*>(p.pt + (size_t)(n_head + d * T + n) * Dp + k);
            }
            const int r = lr + 32 * h;
            As[k4 + 0][r] = a.x; As[k4 + 1][r] = a.y; As[k4 + 2][r] = a.z; As[k4 + 3][r] = a.w;
            Ns[k4 + 0][r] = nn.x; Ns[k4 + 1][r] = nn.y; Ns[k4 + 2][r] = nn.z; Ns[k4 + 3][r] = nn.w;
            Bs[k4 + 0][r] = b.x; Bs[k4 + 1][r] = b.y; Bs[k4 + 2][r] = b.z; Bs[k4 + 3][r] = b.w;
        }
        __syncthreads();
#pragma unroll 4
        for (int kk = 0; kk < BK; ++kk) {
            const float4 a4 = *reinterpret_cast<const float4*>(&As[kk][ty * 4]);
            const float4 n4 = *reinterpret_cast<const float4*>(&Ns[kk][ty * 4]);
            const float4 b4 = *reinterpret_cast<const float4*>(&Bs[kk][tx * 4]);
            const float av[4] = {a4.x, a4.y, a4.z, a4.w};
            const float nv[4] = {n4.x, n4.y, n4.z, n4.w};
            const float bv[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float e = av[i] - (bv[j] - nv[i] * cm[i][j]);  // p - (tail - n c)
                    acc[i][j] += fabsf(e);
                    q[i][j] = fmaf(sign0(e), nv[i], q[i][j]);
                }
        }
        __syncthreads();
    }

    const float Tn = (float)T;
    const float w_pos = uniform_f32(0.5f * Tn), w_neg = uniform_f32((0.5f * Tn) / (float)(T - 1));
    const float inv_norm = uniform_f32(1.f / ((float)sh.S * (float)B * Tn));
    const float grad_scale = uniform_f32(inv_norm * sh.loss_scale);
    float loss_acc = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= B) continue;
        const uint32_t label = OM == 0 ? label_s[ty * 4 + i] : 0u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= T) continue;
            const float score = sh.gamma - acc[i][j];
            float outv = score, dcv = q[i][j];
            if (OM == 0) {
                const bool pos = (uint32_t)n == label;
                const float sign = pos ? 1.f : -1.f, w = pos ? w_pos : w_neg;
                float lsig, dlsig;
                log_sigmoid_both(sign * score, lsig, dlsig);
                loss_acc -= w * lsig;
                outv = w * sign * dlsig * grad_scale;  // d loss / d distance = -d loss / d score
                dcv = outv * q[i][j];
            }
            p.coef[((size_t)d * B + m) * T + n] = outv;
            if (p.dcm) p.dcm[((size_t)d * B + m) * T + n] = dcv;
        }
    }
    if (OM == 0) {
        loss_acc = wave_sum(loss_acc);
        if ((tid & 63) == 0) red[tid >> 6] = loss_acc;
        __syncthreads();
        if (tid == 0) {
            const int n_part = tile.gx * tile.gy;
            p.loss_part[(size_t)d * n_part + tile.y * tile.gx + tile.x] =
                (red[0] + red[1] + red[2] + red[3]) * inv_norm;
        }
    }
}
void launch_transh_fwd(const TranshFwd& p, bool fused_loss, hipStream_t stream) {
    const dim3 grid = tile_grid((p.sh.T + kScoreTile - 1) / kScoreTile, (p.sh.B + kScoreTile - 1) / kScoreTile, p.sh.S);
    if (fused_loss) hipLaunchKernelGGL(k_transh_fwd<0>, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(k_transh_fwd<1>, grid, dim3(256), 0, stream, p);
}

// a[i] *= b[i]
__global__ __launch_bounds__(256) void k_mul_rows(float* __restrict__ a, const float* __restrict__ b, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) a[i] *= b[i];
}
void launch_mul_rows(float* a, const float* b, int64_t n, hipStream_t stream) {
    hipLaunchKernelGGL(k_mul_rows, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, a, b, n);
}

// Backward through the distance, 64 self rows x 64 columns per workgroup, all rows of the
// other side in slabs of 32.  With s = sign(e) and G = coef:
//   SIDE_B false (self = positives):  grad[b]  = sum_t G s          (d loss / d p)
//                                     gn[b]   += sum_t G s c        (added to d c's share, in place)
//   SIDE_B true  (self = tails):      grad[t]  = gt[t] - sum_b G s  (gt = d c's share)
// gn / gt are the rows of `mm` (the dot-product backward on `nt` with coefficient dcm).
template <bool SIDE_B>
__global__ __launch_bounds__(256) void k_transh_bwd(TranshBwd p) {
    __shared__ __attribute__((aligned(16))) float Cs[BJ][LDP];  // G[j][i]
    __shared__ __attribute__((aligned(16))) float Ms[BJ][LDP];  // c[j][i]
    __shared__ __attribute__((aligned(16))) float Os[BJ][LDP];  // other side's main rows [j][k]
    __shared__ __attribute__((aligned(16))) float Qs[SIDE_B ? BJ : 1][LDP];  // other side's normals [j][k]
    const int B = p.B, T = p.T, Dp = p.Dp;
    const int n_self = SIDE_B ? T : B, n_other = SIDE_B ? B : T;
    const TileId tile = xcd_tile((Dp + kScoreTile - 1) / kScoreTile, (n_self + kScoreTile - 1) / kScoreTile, p.S);
    const int d = tile.z, i0 = tile.y * kScoreTile, kt0 = tile.x * kScoreTile;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int n_head = p.S * B;
    const int self_c0 = SIDE_B ? n_head + d * T : d * B, other_c0 = SIDE_B ? d * B : n_head + d * T;
    const float* coef = p.coef + (size_t)d * B * T;
    const float* cmat = p.cmat + (size_t)d * B * T;

    float sv[4][4], sn[4][4], acc[4][4], accn[4][4];
    const int kcol = kt0 + tx * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = i0 + ty * 4 + i;
        float4 v = make_float4(0, 0, 0, 0), n = v;
        if (r < n_self && kcol < Dp) {
            v = *reinterpret_cast<const float4*>(p.pt + (size_t)(self_c0 + r) * Dp + kcol);
            if (!SIDE_B) n = *reinterpret_cast<const float4*>(p.nt + (size_t)(self_c0 + r) * Dp + kcol);
        }
        sv[i][0] = v.x; sv[i][1] = v.y; sv[i][2] = v.z; sv[i][3] = v.w;
        sn[i][0] = n.x; sn[i][1] = n.y; sn[i][2] = n.z; sn[i][3] = n.w;
#pragma unroll
        for (int k = 0; k < 4; ++k) { acc[i][k] = 0.f; accn[i][k] = 0.f; }
    }

    for (int j0 = 0; j0 < n_other; j0 += BJ) {
        for (int idx = tid; idx < BJ * kScoreTile; idx += 256) {
            int i, j;
            size_t at;
            bool live;
            if (!SIDE_B) {  // G[i0 + i][j0 + j], contiguous over j
                j = idx & (BJ - 1); i = idx / BJ;
                live = i0 + i < B && j0 + j < T;
                at = (size_t)(i0 + i) * T + j0 + j;
            } else {        // G[j0 + j][i0 + i], contiguous over i
                i = idx & (kScoreTile - 1); j = idx / kScoreTile;
                live = j0 + j < B && i0 + i < T;
                at = (size_t)(j0 + j) * T + i0 + i;
            }
            Cs[j][i] = live ? coef[at] : 0.f;
            Ms[j][i] = live ? cmat[at] : 0.f;
        }
        {
            const int lj = tid >> 4, kk4 = (tid & 15) * 4;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int j = lj + 16 * h, gj = j0 + j, gk = kt0 + kk4;
                float4 t = make_float4(0, 0, 0, 0), n = t;
                if (gj < n_other && gk < Dp) {
                    t = *reinterpret_cast<const float4*>(p.pt + (size_t)(other_c0 + gj) * Dp + gk);
                    if (SIDE_B) n = *reinterpret_cast<const float4*>(p.nt + (size_t)(other_c0 + gj) * Dp + gk);
                }
                *reinterpret_cast<float4*>(&Os[j][kk4]) = t;
                if (SIDE_B) *reinterpret_cast<float4*>(&Qs[j][kk4]) = n;
            }
        }
        __syncthreads();
#pragma unroll 4
        for (int jj = 0; jj < BJ; ++jj) {
            const float4 c4 = *reinterpret_cast<const float4*>(&Cs[jj][ty * 4]);
            const float4 m4 = *reinterpret_cast<const float4*>(&Ms[jj][ty * 4]);
            const float4 o4 = *reinterpret_cast<const float4*>(&Os[jj][tx * 4]);
            float4 q4 = make_float4(0, 0, 0, 0);
            if (SIDE_B) q4 = *reinterpret_cast<const float4*>(&Qs[jj][tx * 4]);
            const float cv[4] = {c4.x, c4.y, c4.z, c4.w};
            const float mv[4] = {m4.x, m4.y, m4.z, m4.w};
            const float ov[4] = {o4.x, o4.y, o4.z, o4.w};
            const float qv[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (!SIDE_B) {
                        const float g = cv[i] * sign0(sv[i][k] - (ov[k] - sn[i][k] * mv[i]));
                        acc[i][k] += g;
                        accn[i][k] = fmaf(g, mv[i], accn[i][k]);
                    } else {
                        acc[i][k] -= cv[i] * sign0(ov[k] - (sv[i][k] - qv[k] * mv[i]));
                    }
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = i0 + ty * 4 + i;
        if (r >= n_self || kcol >= Dp) continue;
        float* mrow = p.mm + (size_t)(self_c0 + r) * Dp + kcol;
        const float4 add = *reinterpret_cast<const float4*>(mrow);
        float4 out = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
        if (SIDE_B) {
            out = f4add(out, add);
        } else {
            *reinterpret_cast<float4*>(mrow) =
                make_float4(add.x + accn[i][0], add.y + accn[i][1], add.z + accn[i][2], add.w + accn[i][3]);
        }
        *reinterpret_cast<float4*>(p.grad + (size_t)(self_c0 + r) * Dp + kcol) = out;
    }
}
void launch_transh_bwd(const TranshBwd& p, hipStream_t stream) {
    const int gk = (p.Dp + kScoreTile - 1) / kScoreTile;
    hipLaunchKernelGGL(k_transh_bwd<false>, tile_grid(gk, (p.B + kScoreTile - 1) / kScoreTile, p.S), dim3(256), 0,
                       stream, p);
    hipLaunchKernelGGL(k_transh_bwd<true>, tile_grid(gk, (p.T + kScoreTile - 1) / kScoreTile, p.S), dim3(256), 0,
                       stream, p);
}

// Backward through transHPredict, one wave per positive c: from gp = grad[c] (d loss / d p) and
// gn = mm[c] (d loss / d n from the score) to
//   grad[c]            = gp - n (gp . n)                              the head's gradient
//   relgrad[c]         = gp                                           relation embedding row
//   relgrad[n_head+c]  = (g - n (n . g)) / |w|,  g = gn - (n . h) gp - h (gp . n)   normal row
__global__ __launch_bounds__(256) void k_transh_back(RowSource ent, const float* __restrict__ rel,
                                                     const uint32_t* __restrict__ crel, int n_rel, int n_head,
                                                     int Dp, float* __restrict__ grad,
                                                     const float* __restrict__ mm, float* __restrict__ relgrad) {
    const int lane = threadIdx.x & 63;
    const int c = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (c >= n_head) return;
    const float* w = rel + (size_t)(n_rel + crel[c]) * Dp;
    const char* hrow = row_ptr(ent, c);
    float* gp = grad + (size_t)c * Dp;
    const float* gn = mm + (size_t)c * Dp;
    float ss = 0.f;
    for (int k = lane * 4; k < Dp; k += 256) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + k);
        ss += w4.x * w4.x + w4.y * w4.y + w4.z * w4.z + w4.w * w4.w;
    }
    const float nrm = sqrtf(wave_sum(ss));
    float a = 0.f, sgn = 0.f;
    for (int k = lane * 4; k < Dp; k += 256) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + k);
        const float4 h4 = load4(hrow, k, ent);
        const float4 g4 = *reinterpret_cast<const float4*>(gp + k);
        const float n[4] = {w4.x / nrm, w4.y / nrm, w4.z / nrm, w4.w / nrm};
        a += n[0] * h4.x + n[1] * h4.y + n[2] * h4.z + n[3] * h4.w;
        sgn += n[0] * g4.x + n[1] * g4.y + n[2] * g4.z + n[3] * g4.w;
    }
    a = wave_sum(a);
    sgn = wave_sum(sgn);
    float ngn = 0.f;
    for (int k = lane * 4; k < Dp; k += 256) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + k);
        const float4 h4 = load4(hrow, k, ent);
        const float4 g4 = *reinterpret_cast<const float4*>(gp + k);
        const float4 q4 = *reinterpret_cast<const float4*>(gn + k);
        ngn += (w4.x / nrm) * (q4.x - a * g4.x - h4.x * sgn) + (w4.y / nrm) * (q4.y - a * g4.y - h4.y * sgn) +
               (w4.z / nrm) * (q4.z - a * g4.z - h4.z * sgn) + (w4.w / nrm) * (q4.w - a * g4.w - h4.w * sgn);
    }
    ngn = wave_sum(ngn);
    for (int k = lane * 4; k < Dp; k += 256) {
        const float4 w4 = *reinterpret_cast<const float4*>(w + k);
        const float4 h4 = load4(hrow, k, ent);
        const float4 g4 = *reinterpret_cast<const float4*>(gp + k);
        const float4 q4 = *reinterpret_cast<const float4*>(gn + k);
        const float n[4] = {w4.x / nrm, w4.y / nrm, w4.z / nrm, w4.w / nrm};
        const float g[4] = {g4.x, g4.y, g4.z, g4.w}, h[4] = {h4.x, h4.y, h4.z, h4.w}, qq[4] = {q4.x, q4.y, q4.z, q4.w};
        float gh[4], gw[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            gh[x] = g[x] - n[x] * sgn;
            gw[x] = ((qq[x] - a * g[x] - h[x] * sgn) - n[x] * ngn) / nrm;
        }
        *reinterpret_cast<float4*>(relgrad + (size_t)c * Dp + k) = g4;
        *reinterpret_cast<float4*>(relgrad + (size_t)(n_head + c) * Dp + k) = make_float4(gw[0], gw[1], gw[2], gw[3]);
        *reinterpret_cast<float4*>(gp + k) = make_float4(gh[0], gh[1], gh[2], gh[3]);
    }
}
void launch_transh_back(const RowSource& ent, const float* rel, const uint32_t* crel, int n_rel, int n_head,
                        int Dp, float* grad, const float* mm, float* relgrad, hipStream_t stream) {
    hipLaunchKernelGGL(k_transh_back, dim3((n_head + 3) / 4), dim3(256), 0, stream, ent, rel, crel, n_rel, n_head,
                       Dp, grad, mm, relgrad);
}

// --------------------------------------------------------------------------
// Feature MLP (src/poplar_kge.cpp:453-458): per distinct row,
//   hidden = value + relu([value | feature . W] . Up) . Down,   Up [2 Dp, M], Down [M, Dp]
// (device rows of Up: [0, Dp) the embedding's, [Dp, 2 Dp) the projected features').  Plain
// vector kernels, one workgroup per row: written for correctness, no benchmark workload uses it.

// concat[u] = [embedding | fproj[u]], pre[u] = concat . Up, hidden[u] = embedding + relu(pre) . Down
__global__ __launch_bounds__(256) void k_mlp_fwd(MlpArgs a, const float* __restrict__ fproj,
                                                 float* __restrict__ hidden) {
    extern __shared__ float mlp_sm[];
    float* cc = mlp_sm;
    float* boom = mlp_sm + 2 * a.Dp;
    const int u = blockIdx.x, tid = threadIdx.x, Dp = a.Dp, M = a.M;
    if (u >= (int)a.counts[0]) return;
    const char* erow = a.emb_base + (int64_t)a.uniq_key[u] * a.pitch;
    for (int i = tid; i < Dp; i += 256) {
        const float e = load1(erow, i, a.emb_etype), f = fproj[(size_t)u * Dp + i];
        cc[i] = e; cc[Dp + i] = f;
        a.concat[(size_t)u * 2 * Dp + i] = e;
        a.concat[(size_t)u * 2 * Dp + Dp + i] = f;
    }
    __syncthreads();
    for (int m = tid; m < M; m += 256) {
        float acc = 0.f;
        for (int i = 0; i < 2 * Dp; ++i) acc = fmaf(cc[i], a.up[(size_t)i * M + m], acc);
        a.pre[(size_t)u * M + m] = acc;
        boom[m] = fmaxf(acc, 0.f);
    }
    __syncthreads();
    for (int k = tid; k < Dp; k += 256) {
        float acc = 0.f;
        for (int m = 0; m < M; ++m) acc = fmaf(boom[m], a.down[(size_t)m * Dp + k], acc);
        hidden[(size_t)u * Dp + k] = a.add_value ? cc[k] + acc : acc;
    }
}
void launch_mlp_fwd(const MlpArgs& a, const float* fproj, float* hidden, hipStream_t stream) {
    hipLaunchKernelGGL(k_mlp_fwd, dim3(a.max_rows), dim3(256), (size_t)(2 * a.Dp + a.M) * 4, stream, a, fproj,
                       hidden);
}

// From g[u] = d loss / d (MLP output): gpre[u] = (g . Down^T) where pre >= 0 (the reference's max
// passes the gradient where input == output, so also at exactly 0: src/pag/pag.cpp:650-658);
// d concat = gpre . Up^T, whose first half (+ val_add[u], or null) is what the embedding's update
// must add (-> gval) and whose second half is the projected features' gradient (-> gfproj)
__global__ __launch_bounds__(256) void k_mlp_bwd_rows(MlpArgs a, const float* __restrict__ g,
                                                      const float* __restrict__ val_add,
                                                      float* __restrict__ gpre, float* __restrict__ gval,
                                                      float* __restrict__ gfproj) {
    extern __shared__ float mlp_sm[];
    float* gs = mlp_sm;
    float* gp = mlp_sm + a.Dp;
    const int u = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, Dp = a.Dp, M = a.M;
    if (u >= (int)a.counts[0]) return;
    for (int k = tid; k < Dp; k += 256) gs[k] = g[(size_t)u * Dp + k];
    __syncthreads();
    for (int m = wave; m < M; m += 4) {
        float part = 0.f;
        for (int k = lane; k < Dp; k += 64) part = fmaf(gs[k], a.down[(size_t)m * Dp + k], part);
        part = wave_sum(part);
        const float v = a.pre[(size_t)u * M + m] >= 0.f ? part : 0.f;
        if (lane == 0) { gpre[(size_t)u * M + m] = v; gp[m] = v; }
    }
    __syncthreads();
    for (int i = wave; i < 2 * Dp; i += 4) {
        float part = 0.f;
        for (int m = lane; m < M; m += 64) part = fmaf(gp[m], a.up[(size_t)i * M + m], part);
        part = wave_sum(part);
        if (lane == 0) {
            if (i < Dp) gval[(size_t)u * Dp + i] = part + (val_add ? val_add[(size_t)u * Dp + i] : 0.f);
            else gfproj[(size_t)u * Dp + i - Dp] = part;
        }
    }
}
void launch_mlp_bwd_rows(const MlpArgs& a, const float* g, const float* val_add, float* gpre, float* gval,
                         float* gfproj, hipStream_t stream) {
    hipLaunchKernelGGL(k_mlp_bwd_rows, dim3(a.max_rows), dim3(256), (size_t)(a.Dp + a.M) * 4, stream, a, g,
                       val_add, gpre, gval, gfproj);
}

// C[i, n] = sum over rows u < *count, in order, of f(A[u, i]) * B[u, n]; f = max(., 0) with `relu`
__global__ __launch_bounds__(256) void k_rows_atb(const float* __restrict__ A, int lda, int relu,
                                                  const float* __restrict__ B, int ldb, int N,
                                                  const uint32_t* __restrict__ count, float* __restrict__ C) {
    const int i = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    const int U = (int)count[0];
    float acc = 0.f;
    for (int u = 0; u < U; ++u) {
        float x = A[(size_t)u * lda + i];
        if (relu) x = fmaxf(x, 0.f);
        acc = fmaf(x, B[(size_t)u * ldb + n], acc);
    }
    C[(size_t)i * N + n] = acc;
}
void launch_rows_atb(const float* A, int lda, int Ka, bool relu, const float* B, int ldb, int N,
                     const uint32_t* count, float* C, hipStream_t stream) {
    hipLaunchKernelGGL(k_rows_atb, dim3((N + 255) / 256, Ka), dim3(256), 0, stream, A, lda, relu ? 1 : 0, B, ldb,
                       N, count, C);
}

// --------------------------------------------------------------------------
// Feature dropout (src/poplar_kge.cpp:459-461; src/pag/pag.cpp:596-617): the feature part of
// hidden times keep / (1 - p), drawn once for a row's use as a head and once for its use as a
// tail, so a distinct row has two hidden rows: hidden[u] (head use) and hidden[rows + u].
// The keep mask is a hash of (seed, optimiser step, role, table row, column) compared with
// p * 2^32; the reference's device random stream cannot be reproduced, the CPU oracle uses
// this same hash.
DEVINL bool dropout_keep(uint32_t seed, uint32_t step, uint32_t role, uint32_t key, uint32_t k, uint32_t threshold) {
    uint32_t x = key * 0x9E3779B1u + k * 0x85EBCA77u + role * 0xC2B2AE3Du + step * 0x27D4EB2Fu + seed * 0x165667B1u;
    x ^= x >> 16; x *= 0x7FEB352Du; x ^= x >> 15; x *= 0x846CA68Bu; x ^= x >> 16;
    return x >= threshold;
}

// one wave per distinct row: fh_head / fh_tail [max_rows, Dp] = the feature part for either use
// (the same array unless the feature networks are separate), hidden [2 max_rows, Dp]
__global__ __launch_bounds__(256) void k_dropout_hidden(DropoutArgs a, const float* __restrict__ fh_head,
                                                        const float* __restrict__ fh_tail,
                                                        float* __restrict__ hidden) {
    const int lane = threadIdx.x & 63;
    const int u = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= (int)a.counts[0]) return;
    const uint32_t key = a.uniq_key[u];
    const char* erow = a.emb_base + (int64_t)key * a.pitch;
    for (int k = lane * 4; k < a.Dp; k += 256) {
        const float4 v4 = load4(erow, k, a.emb_etype);
        const float4 f4 = *reinterpret_cast<const float4*>(fh_head + (size_t)u * a.Dp + k);
        const float4 t4 = *reinterpret_cast<const float4*>(fh_tail + (size_t)u * a.Dp + k);
        const float v[4] = {v4.x, v4.y, v4.z, v4.w}, f[4] = {f4.x, f4.y, f4.z, f4.w}, ft[4] = {t4.x, t4.y, t4.z, t4.w};
        float oh[4], ot[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            oh[x] = v[x] + (dropout_keep(a.seed, a.step, 0u, key, (uint32_t)(k + x), a.threshold) ? f[x] * a.scale : 0.f);
            ot[x] = v[x] + (dropout_keep(a.seed, a.step, 1u, key, (uint32_t)(k + x), a.threshold) ? ft[x] * a.scale : 0.f);
        }
        *reinterpret_cast<float4*>(hidden + (size_t)u * a.Dp + k) = make_float4(oh[0], oh[1], oh[2], oh[3]);
        *reinterpret_cast<float4*>(hidden + (size_t)(a.max_rows + u) * a.Dp + k) = make_float4(ot[0], ot[1], ot[2], ot[3]);
    }
}
void launch_dropout_hidden(const DropoutArgs& a, const float* fh_head, const float* fh_tail, float* hidden,
                           hipStream_t stream) {
    hipLaunchKernelGGL(k_dropout_hidden, dim3((a.max_rows + 3) / 4), dim3(256), 0, stream, a, fh_head, fh_tail,
                       hidden);
}

// which hidden row contribution c reads: its distinct row, in the tail half for a tail
__global__ __launch_bounds__(256) void k_role_index(const uint32_t* __restrict__ item_row, int n_head, int n,
                                                    uint32_t* __restrict__ out) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c < n) out[c] = item_row[c] + (c >= n_head ? (uint32_t)n : 0u);
}
void launch_role_index(const uint32_t* item_row, int n_head, int n, uint32_t* out, hipStream_t stream) {
    hipLaunchKernelGGL(k_role_index, dim3((n + 255) / 256), dim3(256), 0, stream, item_row, n_head, n, out);
}

// The feature part's gradient per distinct row, one wave per row: its head contributions and its
// tail contributions summed apart (in sorted order).  With dropout (a.enabled) each sum passes
// where that use's dropout output is non-zero (the reference's backward tests the output,
// pag.cpp:610), times 1 / (1 - p).  out_tail null: the two sums go to out_head added up (one
// feature network); else each to its own array (separate networks).
__global__ __launch_bounds__(256) void k_role_sums(DropoutArgs a, ContribSrc cs, const uint32_t* __restrict__ seg_start,
                                                   const uint32_t* __restrict__ seg_real,
                                                   const float* __restrict__ fh_head,
                                                   const float* __restrict__ fh_tail,
                                                   const float* __restrict__ add_head,
                                                   const float* __restrict__ add_tail,
                                                   float* __restrict__ out_head, float* __restrict__ out_tail) {
    const int lane = threadIdx.x & 63;
    const int u = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= (int)a.counts[0]) return;
    const uint32_t key = a.uniq_key[u], pos = seg_start[u], n = seg_real[u];
    for (int k0 = 0; k0 < a.Dp; k0 += 256) {
        const int k = k0 + lane * 4;
        if (k >= a.Dp) continue;
        float4 gh = make_float4(0, 0, 0, 0), gt = gh;
        for (uint32_t j = 0; j < n; ++j) {
            const uint32_t c = cs.sorted_item[pos + j];
            const float4 v = load_contrib<true>(cs, c, k, a.Dp);
            if (c < (uint32_t)cs.n_head) gh = f4add(gh, v); else gt = f4add(gt, v);
        }
        if (add_head) {  // the regularisers' share (of the tensors after dropout)
            gh = f4add(gh, *reinterpret_cast<const float4*>(add_head + (size_t)u * a.Dp + k));
            gt = f4add(gt, *reinterpret_cast<const float4*>(add_tail + (size_t)u * a.Dp + k));
        }
        float h[4] = {gh.x, gh.y, gh.z, gh.w}, t[4] = {gt.x, gt.y, gt.z, gt.w};
        if (a.enabled) {
            const float4 f4 = *reinterpret_cast<const float4*>(fh_head + (size_t)u * a.Dp + k);
            const float4 t4 = *reinterpret_cast<const float4*>(fh_tail + (size_t)u * a.Dp + k);
            const float f[4] = {f4.x, f4.y, f4.z, f4.w}, ft[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const bool kh = f[x] * a.scale != 0.f && dropout_keep(a.seed, a.step, 0u, key, (uint32_t)(k + x), a.threshold);
                const bool kt = ft[x] * a.scale != 0.f && dropout_keep(a.seed, a.step, 1u, key, (uint32_t)(k + x), a.threshold);
                h[x] = kh ? a.scale * h[x] : 0.f;
                t[x] = kt ? a.scale * t[x] : 0.f;
            }
        }
        if (out_tail) {
            *reinterpret_cast<float4*>(out_head + (size_t)u * a.Dp + k) = make_float4(h[0], h[1], h[2], h[3]);
            *reinterpret_cast<float4*>(out_tail + (size_t)u * a.Dp + k) = make_float4(t[0], t[1], t[2], t[3]);
        } else {
            *reinterpret_cast<float4*>(out_head + (size_t)u * a.Dp + k) =
                make_float4(h[0] + t[0], h[1] + t[1], h[2] + t[2], h[3] + t[3]);
        }
    }
}
void launch_role_sums(const DropoutArgs& a, const ContribSrc& cs, const uint32_t* seg_start, const uint32_t* seg_real,
                      const float* fh_head, const float* fh_tail, const float* add_head, const float* add_tail,
                      float* out_head, float* out_tail, hipStream_t stream) {
    hipLaunchKernelGGL(k_role_sums, dim3((a.max_rows + 3) / 4), dim3(256), 0, stream, a, cs, seg_start, seg_real,
                       fh_head, fh_tail, add_head, add_tail, out_head, out_tail);
}

}  // namespace kge
