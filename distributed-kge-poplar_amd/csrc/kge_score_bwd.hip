// gfx950 kernels of the scoring backward pass: l1 / l2distancegrad and the matMul backward
// (src/pag/pag.cpp:685-700, 777-836; the distance codelets of src/poplar_extensions).
#include "kge_device.h"

#include <algorithm>
#include <cstdint>

namespace kge {

// --------------------------------------------------------------------------
// scoring: backward.  out[i, k] = sum_j c[i, j] * phi(self[i, k], other[j, k])
//   L1   phi = signum(self - other)
//   L2   phi = self - other              (c already holds g / dist)
//   DOT  phi = other



template <int DIST>
__global__ __launch_bounds__(256) void k_score_bwd(BwdParams p) {
    __shared__ __attribute__((aligned(16))) float Cs[BJ][LDP];  // Cs[j][i]
    __shared__ __attribute__((aligned(16))) float Os[BJ][LDP];  // Os[j][k]
    const int B = p.B, T = p.T, Dp = p.Dp;
    const int n_self = p.side_b ? T : B;
    const TileId tile = xcd_tile((Dp + kScoreTile - 1) / kScoreTile, (n_self + kScoreTile - 1) / kScoreTile, p.S);
    const int d = tile.z, i0 = tile.y * kScoreTile, kt0 = tile.x * kScoreTile;
    const int t_live = tail_limit(p.tcount, d, T, p.tpad);  // merged tails: the block's live columns
    const int n_other = p.side_b ? B : t_live;
    if (p.side_b && i0 >= t_live) return;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int self_c0 = (p.side_b ? p.b_c0 + d * T : p.a_c0 + d * B);
    const int other_c0 = (p.side_b ? p.a_c0 + d * B : p.b_c0 + d * T);
    const int self_rel = p.side_b ? 0 : p.a_rel_mode, other_rel = p.side_b ? p.a_rel_mode : 0;
    const RowSource& self_src = p.side_b ? p.ent_b : p.ent_a;
    const RowSource& other_src = p.side_b ? p.ent_a : p.ent_b;
    const float* coef = p.coef + (size_t)d * B * T;
    const float* cdiv = p.coef_div ? p.coef_div + (size_t)d * B * T : nullptr;

    // this thread's 4x4 block of `self` (needed by L1 in the loop, by L2 at the end)
    float sv[4][4];
    const int kcol = kt0 + tx * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = i0 + ty * 4 + i;
        float4 v = make_float4(0, 0, 0, 0);
        if (DIST != DIST_DOT && r < n_self && kcol < Dp) {
            v = load4(row_ptr(self_src, self_c0 + r), kcol, self_src);
            if (self_rel) v = combine_rel(v, p.rel + (size_t)p.crel[d * B + r] * Dp, kcol, self_rel);
        }
        sv[i][0] = v.x; sv[i][1] = v.y; sv[i][2] = v.z; sv[i][3] = v.w;
    }
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[i][k] = 0.f;

    for (int j0 = 0; j0 < n_other; j0 += BJ) {
        // coefficient tile -> Cs[j][i]
        if (!p.side_b) {
            // c[i][j] = coef[i0+i][j0+j], contiguous over j: transposing store
            const int li = tid >> 3, j4 = (tid & 7) * 4;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int i = li + 32 * h, gi = i0 + i, gj = j0 + j4;
                float v[4] = {0.f, 0.f, 0.f, 0.f};
                if (gi < B) {
                    const float* src = coef + (size_t)gi * T + gj;
                    if (cdiv) {
                        const float* dv = cdiv + (size_t)gi * T + gj;
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            if (gj + x < T) v[x] = dv[x] != 0.f ? src[x] / dv[x] : 0.f;
                    } else if (gj + 3 < T && (T & 3) == 0) {
                        const float4 t = *reinterpret_cast<const float4*>(src);
                        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
                    } else {
#pragma unroll
                        for (int x = 0; x < 4; ++x) if (gj + x < T) v[x] = src[x];
                    }
                }
#pragma unroll
                for (int x = 0; x < 4; ++x) Cs[j4 + x][i] = v[x];
            }
        } else {
            // c[i][j] = coef[j0+j][i0+i], contiguous over i: direct store
            const int lj = tid >> 4, i4 = (tid & 15) * 4;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int j = lj + 16 * h, gj = j0 + j, gi = i0 + i4;
                float4 t = make_float4(0, 0, 0, 0);
                if (gj < B) {
                    const float* src = coef + (size_t)gj * T + gi;
                    if (cdiv) {
                        const float* dv = cdiv + (size_t)gj * T + gi;
                        if (gi + 0 < T) t.x = dv[0] != 0.f ? src[0] / dv[0] : 0.f;
                        if (gi + 1 < T) t.y = dv[1] != 0.f ? src[1] / dv[1] : 0.f;
                        if (gi + 2 < T) t.z = dv[2] != 0.f ? src[2] / dv[2] : 0.f;
                        if (gi + 3 < T) t.w = dv[3] != 0.f ? src[3] / dv[3] : 0.f;
                    } else if (gi + 3 < T && (T & 3) == 0) {
                        t = *reinterpret_cast<const float4*>(src);
                    } else {
                        if (gi + 0 < T) t.x = src[0];
                        if (gi + 1 < T) t.y = src[1];
                        if (gi + 2 < T) t.z = src[2];
                        if (gi + 3 < T) t.w = src[3];
                    }
                }
                *reinterpret_cast<float4*>(&Cs[j][i4]) = t;
            }
        }
        // other rows -> Os[j][k]
        {
            const int lj = tid >> 4, kk4 = (tid & 15) * 4;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int j = lj + 16 * h, gj = j0 + j, gk = kt0 + kk4;
                float4 t = make_float4(0, 0, 0, 0);
                if (gj < n_other && gk < Dp) {
                    t = load4(row_ptr(other_src, other_c0 + gj), gk, other_src);
                    if (other_rel)
                        t = combine_rel(t, p.rel + (size_t)p.crel[d * B + gj] * Dp, gk, other_rel);
                }
                *reinterpret_cast<float4*>(&Os[j][kk4]) = t;
            }
        }
        __syncthreads();
#pragma unroll 8
        for (int jj = 0; jj < BJ; ++jj) {
            const float4 c4 = *reinterpret_cast<const float4*>(&Cs[jj][ty * 4]);
            const float4 o4 = *reinterpret_cast<const float4*>(&Os[jj][tx * 4]);
            const float cv[4] = {c4.x, c4.y, c4.z, c4.w};
            const float ov[4] = {o4.x, o4.y, o4.z, o4.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    if (DIST == DIST_L1) {
                        const float t = sv[i][k] - ov[k];
                        const float sg = (t > 0.f ? 1.f : 0.f) - (t < 0.f ? 1.f : 0.f);
                        acc[i][k] = fmaf(cv[i], sg, acc[i][k]);
                    } else if (DIST == DIST_L2) {
                        acc[i][k] = fmaf(cv[i], sv[i][k] - ov[k], acc[i][k]);
                    } else {
                        acc[i][k] = fmaf(cv[i], ov[k], acc[i][k]);
                    }
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = i0 + ty * 4 + i;
        if (r >= n_self || kcol >= Dp) continue;
        float o[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            o[k] = acc[i][k];
        }
        float* dst = p.grad + (size_t)(p.grad_c0 + d * n_self + r) * Dp + kcol;
        if (p.vec_out) {
            *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) if (kcol + k < Dp) dst[k] = o[k];
        }
    }
}

// --------------------------------------------------------------------------
// scoring backward on the matrix cores (L2 and dot):
//   out[i,k] = sum_j c[i,j] other[j,k]          (a [I x J] . [J x Dp] product)
//   L2: out[i,k] = self[i,k] * sum_j c[i,j] - that product
// Workgroup tile 128 (self rows) x 64 (embedding columns), waves 2 x 2, each
// wave two 32x32 accumulators; the next chunk of c and `other` is fetched into
// registers while the matrix cores work on the current one.

constexpr int BM_TI = 128, BM_TK = 64, BM_LDK = BM_TK + 4;
// LDS of a backward workgroup: two coefficient tiles (the larger layout: 128 x 36 floats),
// two `other` tiles (32 x 68 floats) and the 128 coefficient row sums
constexpr int kBwdSmemBytes = 2 * (BM_TI * 36 * 4) + 2 * (32 * BM_LDK * 4) + BM_TI * 4;

// BJT = rows of `other` staged per iteration (32 or 128) and NW = waves per
// workgroup (4 or 8), chosen as in the forward kernel.
// ALIGNED: n_self % 128 == 0, n_other % BJT == 0, Dp % 64 == 0, T % 4 == 0,
// dense float32 operands without a relation to apply: branch-free staging loads.
template <int DIST, int SIDE_B, int BJT, bool ALIGNED, int NW>
DEVINL void bwd_mfma_body(const BwdParams& p, const int d, const int tile_x, const int tile_y, char* smem) {
    // Both tiles are float4 copies of global memory.  Head side: Cs[i][j] (the
    // coefficient rows as stored), a lane reads four consecutive j of its row i
    // in one 16-byte LDS read.  Tail side: Cs[j][i] (coefficient rows are the
    // other operand's rows), a lane reads its column i of four rows j.
    constexpr int NT = NW * 64;
    constexpr int AT = 8 / NW;        // 32-row accumulator tiles per wave
    constexpr int NCH = BJT / 32;     // 32-row sub-chunks per iteration
    constexpr int HC = 1024 / NT;     // float4 of a 32 x 128 coefficient sub-tile per thread
    constexpr int HO = 512 / NT;      // float4 of a 32 x 64 `other` sub-tile per thread
    constexpr int CS_ROWS = SIDE_B ? BJT : BM_TI, CS_LD = SIDE_B ? BM_TI + 4 : BJT + 4;
    // two copies of each tile: while the matrix cores work on one slab the next is
    // staged into the other copy, with a single barrier per slab
    typedef float CsTile[CS_ROWS][CS_LD];
    typedef float OsTile[BJT][BM_LDK];
    static_assert(2 * sizeof(CsTile) + 2 * sizeof(OsTile) + BM_TI * 4 <= kBwdSmemBytes, "LDS carve-up");
    CsTile* Cs2 = reinterpret_cast<CsTile*>(smem);
    OsTile* Os2 = reinterpret_cast<OsTile*>(smem + 2 * sizeof(CsTile));
    float* csum_s = reinterpret_cast<float*>(smem + 2 * sizeof(CsTile) + 2 * sizeof(OsTile));
    const int i0 = tile_y * BM_TI, kt0 = tile_x * BM_TK;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * (32 * AT), wk = (wave & 1) * 32;
    const int B = p.B, T = p.T, Dp = p.Dp;
    const int t_live = tail_limit(p.tcount, d, T, p.tpad);  // merged tails: the block's live columns
    const int n_self = SIDE_B ? T : B, n_other = SIDE_B ? B : t_live;
    if (i0 >= (SIDE_B ? t_live : n_self)) return;  // the grid is sized for the longer side
    const int grad_c0 = SIDE_B ? p.b_c0 : p.a_c0;
    const int self_c0 = SIDE_B ? p.b_c0 + d * T : p.a_c0 + d * B;
    const int other_c0 = SIDE_B ? p.a_c0 + d * B : p.b_c0 + d * T;
    const int self_rel = SIDE_B ? 0 : p.a_rel_mode, other_rel = SIDE_B ? p.a_rel_mode : 0;
    const RowSource& self_src = SIDE_B ? p.ent_b : p.ent_a;
    const RowSource& other_src = SIDE_B ? p.ent_a : p.ent_b;
    const float* coef = p.coef + (size_t)d * B * T;

    floatx16 acc[AT];
#pragma unroll
    for (int t = 0; t < AT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][r] = 0.f;
    float cs_acc = 0.f;
    constexpr int NQ = NT / BM_TI, QL = 32 / NQ;  // threads per coefficient row, coefficients per thread and slab
    const int crow = tid & (BM_TI - 1), cq = tid / BM_TI;
    const int kcol = kt0 + wk + (lane & 31);

    // L2: this lane's `self` values, in accumulator layout
    float sv[AT][16];
    if (DIST == DIST_L2) {
#pragma unroll
        for (int t = 0; t < AT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = i0 + wi + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (ALIGNED) {
                    sv[t][r] = reinterpret_cast<const float*>(
                        self_src.base + (int64_t)(self_c0 + i) * self_src.pitch)[kcol];
                    continue;
                }
                float v = 0.f;
                if (i < n_self && kcol < Dp) {
                    v = load1(row_ptr(self_src, self_c0 + i), kcol, self_src.etype);
                    if (self_rel) {
                        const float rv = p.rel[(size_t)p.crel[d * B + i] * Dp + kcol];
                        v = self_rel == 1 ? v + rv : v * rv;
                    }
                }
                sv[t][r] = v;
            }
    }
    // near-identical-pair flags of the (self sub-tile, other chunk) blocks
    const int MT = (B + 31) >> 5, NTL = (T + 31) >> 5;
    const uint32_t* nflag = (DIST == DIST_L2 && p.nearflag) ? p.nearflag + (size_t)d * MT * NTL : nullptr;
    auto flag_of = [&](int i_tile, int j_tile) -> uint32_t {
        if (!nflag) return 0u;
        const int mt = SIDE_B ? j_tile : i_tile, nt = SIDE_B ? i_tile : j_tile;
        if (32 * nt >= t_live) return 0u;  // columns the forward pass did not visit
        if (ALIGNED) return nflag[(size_t)mt * NTL + nt];
        return (mt < MT && nt < NTL) ? nflag[(size_t)mt * NTL + nt] : 0u;
    };
    uint32_t nf_next[NCH][AT], nf_row_next[NCH];
    floatx4 creg[NCH][HC], oreg[NCH][HO];
    auto prefetch = [&](int jbase) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int j0 = jbase + 32 * c;
#pragma unroll
            for (int t = 0; t < AT; ++t) nf_next[c][t] = flag_of((i0 + wi + 32 * t) >> 5, j0 >> 5);
            nf_row_next[c] = flag_of((i0 + (tid & (BM_TI - 1))) >> 5, j0 >> 5);
            if constexpr (ALIGNED) {
#pragma unroll
                for (int h = 0; h < HC; ++h) {
                    const int idx = tid + NT * h;
                    const float* src = SIDE_B ? coef + (size_t)(j0 + (idx >> 5)) * T + i0 + (idx & 31) * 4
                                              : coef + (size_t)(i0 + (idx >> 3)) * T + j0 + (idx & 7) * 4;
                    creg[c][h] = *reinterpret_cast<const floatx4*>(src);
                }
#pragma unroll
                for (int h = 0; h < HO; ++h) {
                    const int idx = tid + NT * h;
                    oreg[c][h] = *reinterpret_cast<const floatx4*>(
                        other_src.base + (int64_t)(other_c0 + j0 + (idx >> 4)) * other_src.pitch +
                        (size_t)(kt0 + (idx & 15) * 4) * 4);
                }
            } else {
#pragma unroll
            for (int h = 0; h < HC; ++h) {
                const int idx = tid + NT * h;
                creg[c][h] = floatx4{0.f, 0.f, 0.f, 0.f};
                if (!SIDE_B) {  // c[i][j] = coef[i0+i][j0+j]: float4 along j
                    const int gi = i0 + (idx >> 3), gj = j0 + (idx & 7) * 4;
                    if (gi < B && gj < T) {
                        const float* src = coef + (size_t)gi * T + gj;
                        if (gj + 3 < T && (T & 3) == 0) creg[c][h] = *reinterpret_cast<const floatx4*>(src);
                        else {
                            creg[c][h].x = src[0];
                            if (gj + 1 < T) creg[c][h].y = src[1];
                            if (gj + 2 < T) creg[c][h].z = src[2];
                            if (gj + 3 < T) creg[c][h].w = src[3];
                        }
                    }
                } else {        // c[i][j] = coef[j0+j][i0+i]: float4 along i
                    const int gj = j0 + (idx >> 5), gi = i0 + (idx & 31) * 4;
                    if (gj < B && gi < T) {
                        const float* src = coef + (size_t)gj * T + gi;
                        if (gi + 3 < T && (T & 3) == 0) creg[c][h] = *reinterpret_cast<const floatx4*>(src);
                        else {
                            creg[c][h].x = src[0];
                            if (gi + 1 < T) creg[c][h].y = src[1];
                            if (gi + 2 < T) creg[c][h].z = src[2];
                            if (gi + 3 < T) creg[c][h].w = src[3];
                        }
                    }
                }
            }
#pragma unroll
            for (int h = 0; h < HO; ++h) {
                const int idx = tid + NT * h;
                const int gj = j0 + (idx >> 4), gk = kt0 + (idx & 15) * 4;
                oreg[c][h] = floatx4{0.f, 0.f, 0.f, 0.f};
                if (gj < n_other && gk < Dp) {
                    oreg[c][h] = as_x4(load4(row_ptr(other_src, other_c0 + gj), gk, other_src));
                    if (other_rel)
                        oreg[c][h] = as_x4(combine_rel(as_f4(oreg[c][h]), p.rel + (size_t)p.crel[d * B + gj] * Dp, gk, other_rel));
                }
            }
            }
        }
    };
    bool direct_next[NCH][AT], direct_row_next[NCH], any_direct_next[NCH];
    // writes the prefetched slab into tile copy `nb` and latches its near-pair flags
    auto stage = [&](int nb) __attribute__((always_inline)) {
        CsTile& Cn = Cs2[nb];
        OsTile& On = Os2[nb];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            any_direct_next[c] = false;
#pragma unroll
            for (int t = 0; t < AT; ++t) {
                direct_next[c][t] = nf_next[c][t] != 0u;
                any_direct_next[c] = any_direct_next[c] || direct_next[c][t];
            }
            direct_row_next[c] = nf_row_next[c] != 0u;
#pragma unroll
            for (int h = 0; h < HC; ++h) {
                const int idx = tid + NT * h;
                if (!SIDE_B) {
                    *reinterpret_cast<floatx4*>(&Cn[idx >> 3][32 * c + (idx & 7) * 4]) = creg[c][h];
                } else {
                    *reinterpret_cast<floatx4*>(&Cn[32 * c + (idx >> 5)][(idx & 31) * 4]) = creg[c][h];
                }
            }
#pragma unroll
            for (int h = 0; h < HO; ++h) {
                const int idx = tid + NT * h;
                *reinterpret_cast<floatx4*>(&On[32 * c + (idx >> 4)][(idx & 15) * 4]) = oreg[c][h];
            }
        }
    };
    prefetch(0);
    stage(0);
    __syncthreads();
    if (BJT < n_other) prefetch(BJT);
    for (int jbase = 0, buf = 0; jbase < n_other; jbase += BJT, buf ^= 1) {
        bool direct[NCH][AT], direct_row[NCH], any_direct[NCH];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            any_direct[c] = any_direct_next[c];
            direct_row[c] = direct_row_next[c];
#pragma unroll
            for (int t = 0; t < AT; ++t) direct[c][t] = direct_next[c][t];
        }
        if (jbase + BJT < n_other) {
            stage(buf ^ 1);  // the other copy: last read one slab ago, before the barrier
            if (jbase + 2 * BJT < n_other) prefetch(jbase + 2 * BJT);
        }
        const CsTile& Cc = Cs2[buf];
        const OsTile& Oc = Os2[buf];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int jo = 32 * c;
            // coefficient row sums (L2): NQ threads share a row, each adds its QL of the slab's
            // 32 coefficients, so that every wave carries the same small load
            if (DIST == DIST_L2 && !direct_row[c]) {
                if (SIDE_B) {
#pragma unroll
                    for (int jj = 0; jj < QL; ++jj) cs_acc += Cc[jo + cq * QL + jj][crow];
                } else {
#pragma unroll
                    for (int jj = 0; jj < QL; jj += 4) {
                        const float4 v = *reinterpret_cast<const float4*>(&Cc[crow][jo + cq * QL + jj]);
                        cs_acc += v.x; cs_acc += v.y; cs_acc += v.z; cs_acc += v.w;
                    }
                }
            }
            if (!any_direct[c]) {
                // group g covers rows j = jo + 8g .. 8g+7 of `other`: instruction x
                // takes row 8g + x (lower half-wave) and 8g + 4 + x (upper)
                float ra[2][AT][4], rb[2][4];
                const int hl = lane >> 5, cl = lane & 31;
                auto fetch = [&](int buf, int g) {
#pragma unroll
                    for (int x = 0; x < 4; ++x) rb[buf][x] = Oc[jo + 8 * g + 4 * hl + x][wk + cl];
#pragma unroll
                    for (int t = 0; t < AT; ++t) {
                        if (SIDE_B) {
#pragma unroll
                            for (int x = 0; x < 4; ++x) ra[buf][t][x] = Cc[jo + 8 * g + 4 * hl + x][wi + 32 * t + cl];
                        } else {
                            const float4 v = *reinterpret_cast<const float4*>(&Cc[wi + 32 * t + cl][jo + 8 * g + 4 * hl]);
                            ra[buf][t][0] = v.x; ra[buf][t][1] = v.y; ra[buf][t][2] = v.z; ra[buf][t][3] = v.w;
                        }
                    }
                };
                fetch(0, 0);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    if (g + 1 < 4) fetch((g + 1) & 1, g + 1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int x = 0; x < 4; ++x)
#pragma unroll
                        for (int t = 0; t < AT; ++t)
                            acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[g & 1][t][x], rb[g & 1][x], acc[t], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                // some pair of this block is nearly identical: c * (self - other) directly,
                // as the reference codelet does (acc holds the negated sum, see the epilogue)
#pragma unroll
                for (int t = 0; t < AT; ++t) {
                    if (direct[c][t]) {
                        for (int jj = jo; jj < jo + 32; ++jj) {
                            const float o = Oc[jj][wk + (lane & 31)];
#pragma unroll
                            for (int r = 0; r < 16; ++r) {
                                const int il = wi + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                                const float cc = SIDE_B ? Cc[jj][il] : Cc[il][jj];
                                acc[t][r] = fmaf(-cc, sv[t][r] - o, acc[t][r]);
                            }
                        }
                    } else {
#pragma unroll
                        for (int q = 0; q < 16; ++q) {
                            const int jj = jo + 2 * q + (lane >> 5);
                            const float b = Oc[jj][wk + (lane & 31)];
                            const float a = SIDE_B ? Cc[jj][wi + 32 * t + (lane & 31)] : Cc[wi + 32 * t + (lane & 31)][jj];
                            acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[t], 0, 0, 0);
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
    if (DIST == DIST_L2) {
        // the NQ partial sums of a row, added in a fixed order (the tiles are no longer read)
        float* part = reinterpret_cast<float*>(smem);
        part[cq * BM_TI + crow] = cs_acc;
        __syncthreads();
        if (tid < BM_TI) {
            float sum = part[tid];
#pragma unroll
            for (int q = 1; q < NQ; ++q) sum += part[q * BM_TI + tid];
            csum_s[tid] = sum;
        }
        __syncthreads();
    }
    float* __restrict__ const gout = p.grad;
    if (DIST == DIST_DOT && p.add_base) {
        // added rows: all row ids, then all values, then the stores, so that a tile's loads are
        // in flight together instead of sixteen dependent round trips one after the other
        const char* __restrict__ const ab = p.add_base;
        const uint32_t* __restrict__ const ai = p.add_index;
        const uint32_t cnt = *p.add_count;
#pragma unroll
        for (int t = 0; t < AT; ++t) {
            uint32_t row[16];
            float addv[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = i0 + wi + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                row[r] = ((ALIGNED || i < n_self) && (uint32_t)i < cnt) ? ai[i] : 0u;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r)
                addv[r] = (ALIGNED || kcol < Dp) ? load1(ab + (int64_t)row[r] * p.add_pitch, kcol, p.add_etype) : 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = i0 + wi + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (!ALIGNED && (i >= n_self || kcol >= Dp)) continue;
                gout[(size_t)(grad_c0 + d * n_self + i) * Dp + kcol] = acc[t][r] + addv[r];
            }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < AT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i_loc = wi + 32 * t + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
            const int i = i0 + i_loc;
            if (!ALIGNED && (i >= n_self || kcol >= Dp)) continue;
            float o = acc[t][r];
            if (DIST == DIST_L2) o = sv[t][r] * csum_s[i_loc] - o;
            gout[(size_t)(grad_c0 + d * n_self + i) * Dp + kcol] = o;
        }
}

// one side per launch (p.side_b), or both sides in one launch
template <int DIST, int SIDE_B, int BJT, bool ALIGNED, int NW>
__global__ __launch_bounds__(NW * 64) void k_score_bwd_mfma(BwdParams p) {
    __shared__ __attribute__((aligned(16))) char smem[kBwdSmemBytes];
    const int n_self = SIDE_B ? p.T : p.B;
    const TileId tile = xcd_tile((p.Dp + BM_TK - 1) / BM_TK, (n_self + BM_TI - 1) / BM_TI, p.S);
    bwd_mfma_body<DIST, SIDE_B, BJT, ALIGNED, NW>(p, tile.z, tile.x, tile.y, smem);
}
template <int DIST, int BJT, bool ALIGNED, int NW>
__global__ __launch_bounds__(NW * 64) void k_score_bwd_mfma_both(BwdParams p) {
    __shared__ __attribute__((aligned(16))) char smem[kBwdSmemBytes];  // one allocation serves either side
    // One launch for both sides. The side whose tiles loop over more rows of the other side comes
    // first, for every block, then the other side: the long tiles do not start last (at the end of
    // the launch the CUs run dry while the longest tiles finish), and no workgroup is started for
    // a tile that does not exist. A block's tiles of one side stay together on one XCD; its two
    // sides no longer run close enough in time to share the L2's copy of the operand rows and the
    // coefficient matrix, which was measured to cost less than the late long tiles did.
    const int gx = p.Dp / BM_TK, ga = p.B / BM_TI, gb = p.T / BM_TI;
    const bool heads_first = p.T >= p.B;  // a head tile loops over T rows, a tail tile over B
    const int n_first = gx * (heads_first ? ga : gb) * p.S;
    const int L = blockIdx.x;
    if ((L < n_first) == heads_first) {
        const TileId tile = xcd_tile(gx, ga, p.S, heads_first ? L : L - n_first);
        bwd_mfma_body<DIST, 0, BJT, ALIGNED, NW>(p, tile.z, tile.x, tile.y, smem);
    } else {
        const TileId tile = xcd_tile(gx, gb, p.S, heads_first ? L - n_first : L);
        bwd_mfma_body<DIST, 1, BJT, ALIGNED, NW>(p, tile.z, tile.x, tile.y, smem);
    }
}

// --------------------------------------------------------------------------
// The same sums from bfloat16 matrix instructions on three-piece operands (mfma_split6: six
// v_mfma_f32_32x32x16_bf16 per sixteen rows of `other` in place of eight
// v_mfma_f32_32x32x2_f32, float32 accuracy).  The sum runs over the rows of `other`, so both
// operand tiles are laid down in LDS with that index innermost, as pieces:
//   Ap[piece][self row][32 j]    Bp[piece][embedding column][32 j]
// A thread stages eight consecutive j of one coefficient row (head side: two 16-byte loads along
// the row; tail side: eight 4-byte loads down a column of the coefficient matrix, consecutive
// lanes on consecutive columns) and four consecutive j of one embedding column of `other`.
// A row's four 16-byte chunks sit at position chunk ^ ((row / 4) % 4), which spreads sixteen
// consecutive rows' accesses to one chunk over all banks.
// Workgroup tile 128 (self rows) x 64 (embedding columns), eight waves as 4 x 2, one 32 x 32
// accumulator each; tile-aligned shapes and dense float32 operands only.

constexpr int BS_TI = 128, BS_TK = 64, BS_KJ = 32;
constexpr int kBwdSplitSmemBytes = 2 * 3 * BS_TI * BS_KJ * 2 + 2 * 3 * BS_TK * BS_KJ * 2 + 4 * BS_TI * 4 + BS_TI * 4;

template <int DIST, int SIDE_B>
DEVINL void bwd_split_body(const BwdParams& p, const int d, const int tile_x, const int tile_y, char* smem) {
    typedef uint16_t ATile[3][BS_TI][BS_KJ];
    typedef uint16_t BTile[3][BS_TK][BS_KJ];
    ATile* Ap = reinterpret_cast<ATile*>(smem);
    BTile* Bp = reinterpret_cast<BTile*>(smem + 2 * sizeof(ATile));
    float* part = reinterpret_cast<float*>(smem + 2 * sizeof(ATile) + 2 * sizeof(BTile));  // [4][128]
    float* csum_s = part + 4 * BS_TI;
    const int i0 = tile_y * BS_TI, kt0 = tile_x * BS_TK;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hl = lane >> 5, cl = lane & 31;
    const int wi = (wave >> 1) * 32, wk = (wave & 1) * 32;
    const int B = p.B, T = p.T, Dp = p.Dp;
    const int t_live = tail_limit(p.tcount, d, T, p.tpad);  // merged tails: the block's live columns
    const int n_self = SIDE_B ? T : B, n_other = SIDE_B ? B : t_live;
    if (i0 >= (SIDE_B ? t_live : n_self)) return;  // the grid is sized for the longer side
    const int grad_c0 = SIDE_B ? p.b_c0 : p.a_c0;
    const RowSource& self_src = SIDE_B ? p.ent_b : p.ent_a;
    const RowSource& other_src = SIDE_B ? p.ent_a : p.ent_b;
    const char* const self_rows = self_src.base + (int64_t)(SIDE_B ? p.b_c0 + d * T : p.a_c0 + d * B) * self_src.pitch;
    const char* const other_rows = other_src.base + (int64_t)(SIDE_B ? p.a_c0 + d * B : p.b_c0 + d * T) * other_src.pitch;
    const int64_t opitch = other_src.pitch;
    const float* const coef = p.coef + (size_t)d * B * T;
    const int kcol = kt0 + wk + cl;

    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    // L2: this lane's `self` values, in accumulator layout (fetched where they are used: held
    // through the loop they would cost the registers of a fourth wave per SIMD)
    auto load_self = [&](float sv[16]) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i = i0 + wi + 8 * (r >> 2) + 4 * hl + (r & 3);
            sv[r] = reinterpret_cast<const float*>(self_rows + (int64_t)i * self_src.pitch)[kcol];
        }
    };
    // staging: coefficient row a_row, its j-chunk a_kg (8 values); column b_n of `other`, rows
    // 8 b_kg + 4 b_half .. + 3 of the slab.  What is the same for a whole wave stays in scalar
    // registers, so that the loads take a scalar base and one 32-bit lane offset.
    const int a_row = SIDE_B ? (wave & 1) * 64 + lane : wave * 16 + (lane >> 2), a_kg = SIDE_B ? (wave >> 1) : (lane & 3);
    const int b_n = lane, b_kg = wave & 3, b_half = wave >> 2;
    const int a_col = (a_kg ^ ((a_row >> 2) & 3)) << 3;
    const int b_col = ((b_kg ^ ((b_n >> 2) & 3)) << 3) + 4 * b_half;
    const uint32_t a_off = SIDE_B ? (uint32_t)a_row : (uint32_t)(a_row * T + 8 * a_kg);
    // near-identical-pair flags of the (self sub-tile, slab of `other`) blocks (L2: the forward
    // pass wrote them for the columns it visited)
    const int MT = B >> 5, NTL = T >> 5;
    const uint32_t* const nflag = DIST == DIST_L2 ? p.nearflag + (size_t)d * MT * NTL : nullptr;
    auto flag_of = [&](int i_tile, int j_tile) -> uint32_t {
        if constexpr (DIST != DIST_L2) return 0u;
        const int mt = SIDE_B ? j_tile : i_tile, nt = SIDE_B ? i_tile : j_tile;
        const uint32_t f = nflag[(size_t)mt * NTL + min(nt, NTL - 1)];
        return 32 * nt < t_live ? f : 0u;  // no flags for columns the forward pass did not visit
    };
    float cs_acc = 0.f;
    uint32_t flag_seen = 0u;  // any flagged block among those this thread staged
    // a slab's operand loads take a round trip to the memory-side cache however little work a
    // slab is: two register sets, each filled two slabs ahead of its use
    struct Slab {
        floatx4 a[2], b;
        uint32_t nf_row;
    } set0, set1;
    auto prefetch = [&](Slab& s, int j_first) __attribute__((always_inline)) {
        // (taken through a scalar register afresh: the row addresses are then formed by scalar
        // instructions every slab, not carried along as one 64-bit vector pointer per row)
        const int j0 = __builtin_amdgcn_readfirstlane(j_first);
        s.nf_row = flag_of((i0 + a_row) >> 5, j0 >> 5);
        if (!SIDE_B) {
            const float* src = coef + (size_t)i0 * T + j0;
            s.a[0] = *reinterpret_cast<const floatx4*>(src + a_off);
            s.a[1] = *reinterpret_cast<const floatx4*>(src + a_off + 4);
        } else {
#pragma unroll
            for (int x = 0; x < 8; ++x) s.a[x >> 2][x & 3] = (coef + (size_t)(j0 + 8 * a_kg + x) * T + i0)[a_off];
        }
#pragma unroll
        for (int x = 0; x < 4; ++x)
            s.b[x] = (reinterpret_cast<const float*>(other_rows + (int64_t)(j0 + 8 * b_kg + 4 * b_half + x) * opitch) + kt0)[b_n];
    };
    // writes a prefetched slab into tile copy `nb` as pieces and adds the coefficients to the row
    // sums.  `keep` = 0 for a slab past the end and where some pair of the row's 32 x 32 block is
    // nearly identical: such a block's coefficients go into the tile as zeros (its products
    // vanish, its rows' sums leave it out) and it is taken in the direct form after the loop.
    auto stage = [&](const Slab& s, int nb, float live) __attribute__((always_inline)) {
        const float keep = s.nf_row == 0u ? live : 0.f;
        flag_seen |= s.nf_row;
        const floatx4 a0 = s.a[0] * keep, a1 = s.a[1] * keep;
        uint2 lo[3], hi[3];
        split4_bf16(a0, lo);
        split4_bf16(a1, hi);
#pragma unroll
        for (int q = 0; q < 3; ++q)
            *reinterpret_cast<uint4*>(&Ap[nb][q][a_row][a_col]) = make_uint4(lo[q].x, lo[q].y, hi[q].x, hi[q].y);
        if (DIST == DIST_L2) {
            const floatx4 s4 = a0 + a1;
            cs_acc += (s4.x + s4.y) + (s4.z + s4.w);
        }
        uint2 pb[3];
        split4_bf16(s.b, pb);
#pragma unroll
        for (int q = 0; q < 3; ++q) *reinterpret_cast<uint2*>(&Bp[nb][q][b_n][b_col]) = pb[q];
    };
    const int j_last = n_other - BS_KJ;  // loads past the end fetch the last slab again
    // one slab: the matrix work on tile copy `buf`, the next slab (register set `s`) into the
    // other copy (last read one slab ago, before the barrier), and `s` filled again
    auto step = [&](Slab& s, int jbase, int buf) __attribute__((always_inline)) {
        // two steps of sixteen rows of `other`; a lane supplies rows 8 * (lane / 32) .. + 7 of a
        // step, for its self row and for its embedding column
        floatx4 fa[2][3], fb[2][3];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int chunk = 2 * ks + hl;
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                const int ra = wi + cl, rb = wk + cl;
                fa[ks][q] = *reinterpret_cast<const floatx4*>(&Ap[buf][q][ra][(chunk ^ ((ra >> 2) & 3)) << 3]);
                fb[ks][q] = *reinterpret_cast<const floatx4*>(&Bp[buf][q][rb][(chunk ^ ((rb >> 2) & 3)) << 3]);
            }
        }
        stage(s, buf ^ 1, jbase + BS_KJ < n_other ? 1.f : 0.f);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) acc = mfma_split6(fa[ks], fb[ks], acc);
        // the order asked of the scheduler: the first step's LDS reads, then one matrix
        // instruction (each depends on the one before it), a share of the vector work and an LDS
        // access, in turn
        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
        for (int i = 0; i < 12; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
            if (i < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            else __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
        prefetch(s, min(jbase + 3 * BS_KJ, j_last));
        __syncthreads();
    };
    prefetch(set0, 0);
    stage(set0, 0, 1.f);
    prefetch(set0, min(BS_KJ, j_last));
    prefetch(set1, min(2 * BS_KJ, j_last));
    __syncthreads();
    for (int jbase = 0; jbase < n_other; jbase += 2 * BS_KJ) {  // n_other % 64 == 0
        step(set0, jbase, 0);
        step(set1, jbase + BS_KJ, 1);
    }
    float sv[16];
    if (DIST == DIST_L2) {
        load_self(sv);  // (in flight across the barriers below)
        // the four partial sums of a row, added in a fixed order; and whether any block of the
        // tile was flagged at all
        part[a_kg * BS_TI + a_row] = cs_acc;
        const int any_flag = __syncthreads_or(flag_seen != 0u);
        if (tid < BS_TI) csum_s[tid] = ((part[tid] + part[BS_TI + tid]) + part[2 * BS_TI + tid]) + part[3 * BS_TI + tid];
        __syncthreads();
        // slabs in which some pair of this wave's sub-tile is nearly identical: c * (self - other)
        // directly, as the reference codelet does, from the operands in memory (acc holds the
        // negated sum).  Rare, and out of the loop above so that its registers stay out of it.
        if (any_flag)
            for (int jbase = 0; jbase < n_other; jbase += BS_KJ) {
                if (flag_of((i0 + wi) >> 5, jbase >> 5) == 0u) continue;
                for (int jj = jbase; jj < jbase + BS_KJ; ++jj) {
                    const float o = reinterpret_cast<const float*>(other_rows + (int64_t)jj * opitch)[kcol];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int i = i0 + wi + 8 * (r >> 2) + 4 * hl + (r & 3);
                        const float cc = SIDE_B ? coef[(size_t)jj * T + i] : coef[(size_t)i * T + jj];
                        acc[r] = fmaf(-cc, sv[r] - o, acc[r]);
                    }
                }
            }
    }
    float* __restrict__ const gout = p.grad;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int i_loc = wi + 8 * (r >> 2) + 4 * hl + (r & 3);
        float o = acc[r];
        if (DIST == DIST_L2) o = sv[r] * csum_s[i_loc] - o;
        gout[(size_t)(grad_c0 + d * n_self + i0 + i_loc) * Dp + kcol] = o;
    }
}

// both sides in one launch, in the order of k_score_bwd_mfma_both
template <int DIST>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void k_score_bwd_split_both(BwdParams p) {
    __shared__ __attribute__((aligned(16))) char smem[kBwdSplitSmemBytes];
    const int gx = p.Dp / BS_TK, ga = p.B / BS_TI, gb = p.T / BS_TI;
    const bool heads_first = p.T >= p.B;  // a head tile loops over T rows, a tail tile over B
    const int n_first = gx * (heads_first ? ga : gb) * p.S;
    const int L = blockIdx.x;
    if ((L < n_first) == heads_first) {
        const TileId tile = xcd_tile(gx, ga, p.S, heads_first ? L : L - n_first);
        bwd_split_body<DIST, 0>(p, tile.z, tile.x, tile.y, smem);
    } else {
        const TileId tile = xcd_tile(gx, gb, p.S, heads_first ? L - n_first : L);
        bwd_split_body<DIST, 1>(p, tile.z, tile.x, tile.y, smem);
    }
}

void launch_bwd(const BwdParams& p, int dist_fn, hipStream_t stream) {
    const int n_self = p.side_b ? p.T : p.B;
    const bool mfma_ok = p.use_mfma && !p.coef_div && p.ent_a.vec && p.ent_b.vec && (p.Dp & 3) == 0 &&
                         (dist_fn == DIST_DOT || (dist_fn == DIST_L2 && p.nearflag));
    if (mfma_ok) {
        const dim3 grid = tile_grid((p.Dp + BM_TK - 1) / BM_TK, (n_self + BM_TI - 1) / BM_TI, p.S);
        const int n_other = p.side_b ? p.B : p.T;
        const bool plain = p.ent_a.etype == ET_F32 && p.ent_b.etype == ET_F32 && !p.ent_a.index &&
                           !p.ent_b.index && p.a_rel_mode == 0;
        const bool aligned = plain && n_self % BM_TI == 0 && p.Dp % BM_TK == 0 && p.T % 4 == 0 && n_other % 32 == 0;
#define KGE_BWD(D_, S_)                                                                                     \
    do {                                                                                                    \
        if (aligned) hipLaunchKernelGGL((k_score_bwd_mfma<D_, S_, 32, true, 8>), grid, dim3(512), 0, stream, p); \
        else hipLaunchKernelGGL((k_score_bwd_mfma<D_, S_, 32, false, 4>), grid, dim3(256), 0, stream, p);    \
    } while (0)
        if (dist_fn == DIST_L2) {
            if (p.side_b) KGE_BWD(DIST_L2, 1); else KGE_BWD(DIST_L2, 0);
        } else {
            if (p.side_b) KGE_BWD(DIST_DOT, 1); else KGE_BWD(DIST_DOT, 0);
        }
#undef KGE_BWD
        return;
    }
    const dim3 grid = tile_grid((p.Dp + kScoreTile - 1) / kScoreTile, (n_self + kScoreTile - 1) / kScoreTile, p.S);
    if (dist_fn == DIST_L1)
        hipLaunchKernelGGL(k_score_bwd<DIST_L1>, grid, dim3(256), 0, stream, p);
    else if (dist_fn == DIST_L2)
        hipLaunchKernelGGL(k_score_bwd<DIST_L2>, grid, dim3(256), 0, stream, p);
    else
        hipLaunchKernelGGL(k_score_bwd<DIST_DOT>, grid, dim3(256), 0, stream, p);
}


// --------------------------------------------------------------------------
// L1 backward, both sides in one pass over the pairs.  c * signum(a - b) has no
// contraction form, so this is vector-ALU work; computing the term once and
// adding it to the head's sum and (negated) to the tail's sum halves it.
// One workgroup of 16 waves per (block, 64-column slice); a lane owns one
// column.  Wave w keeps tails [w*tw, (w+1)*tw) and their gradient sums in
// registers and walks over all heads; a head's sum over one wave's tails is a
// partial, the 16 partials of a head meet in LDS and are added in wave order
// (deterministic).  The coefficients of a (head, tail range) are the same for
// every lane: the workgroup stages the coefficient rows of eight heads at a time
// in LDS (one 16-byte load per thread, the next chunk's in flight under the
// current one's arithmetic) and every wave reads its four at a time with one
// LDS instruction whose lanes all name the same address (a broadcast, no bank
// conflict).  As scalar loads (wave-uniform operands straight from memory) the
// same coefficients bounded the kernel: each of a block's four column slices
// pulled the whole coefficient matrix through the scalar caches.
constexpr int L1P_CB = 8;      // heads per chunk
constexpr int L1P_WAVES = 16;

constexpr int L1P_MAX_T = 512;  // tails per block at most (32 per wave)

// the work of one wave with exactly TW tails (TW even): straight-line code over
// its tails, their values and sums in registers.
// signum(a - b) with signum(0) = 0 (poplar_extensions l1distance.codelet.cpp:76-79) from
// instructions of the fast class only (subtract, fused multiply-add): the difference times 2^126
// plus one half, clamped to [0, 1] by the instruction's own output modifier, is p = 1 / 0.5 / 0
// for a positive / zero / negative difference (any normal float times 2^126 is at least 1 in
// magnitude), and signum = 2 p - 1.  The inner loop accumulates c p (four instructions per pair
// and column: subtract, clamped fma, one fma for either side's sum) and the linear part is taken
// off in small pieces, before the sums grow and rounding with them:
//   tails   after every chunk of 8 heads, half the chunk's column sums: the running value is
//           sum c (p - 1/2) = (1/2) sum c signum;
//   heads   each wave's partial 2 sum_j c p minus the sum of the coefficients of its own TW
//           columns, before the 16 waves' values are added.
// The column and row-part sums of a chunk come from the coefficient rows staged in LDS, by waves
// 8 .. 15 while waves 0 .. 7 add the head partials of the chunk before.
template <int TW>
DEVINL void l1_pair_wave(const float* __restrict__ a_rows, const float* __restrict__ b_rows,
                         const float* __restrict__ cblk, float* __restrict__ grad_a, float* __restrict__ grad_b,
                         int B, int T, int Dp, int t_live, int w, int lane,
                         float (*part)[L1P_WAVES][L1P_CB][64], float (*cs)[L1P_CB][L1P_MAX_T],
                         float (*col_half)[L1P_MAX_T], float (*row_part)[L1P_CB][L1P_WAVES]) {
    // In LDS a wave's TW columns start at a multiple of four (TWS apart): its reads stay 16-byte
    // ones when TW is not a multiple of four.  Column c lies at lds_col(c).
    constexpr int TWS = (TW + 3) & ~3;
    auto lds_col = [](int c) { return (c / TW) * TWS + c % TW; };
    const int tid = threadIdx.x, t4 = t_live / 4, l0 = w * TWS;
    // staging: thread -> (head, four columns) of a chunk's coefficient rows, stored as two pairs
    // (TW is even, so a pair never straddles two waves' columns)
    const bool stager = tid < L1P_CB * t4;
    const int s_head = tid / t4, s_col = (tid - s_head * t4) * 4;
    const int s_lo = lds_col(s_col), s_hi = lds_col(s_col + 2);
    auto stage = [&](int buf, float4 v) __attribute__((always_inline)) {
        *reinterpret_cast<float2*>(&cs[buf][s_head][s_lo]) = make_float2(v.x, v.y);
        *reinterpret_cast<float2*>(&cs[buf][s_head][s_hi]) = make_float2(v.z, v.w);
    };
    // linear parts: thread 512 + t -> column t; threads 512 .. 639 -> (head, wave)
    const int u = tid - 512, u_lds = u >= 0 ? lds_col(u) : 0;
    float4 c_next = make_float4(0.f, 0.f, 0.f, 0.f);
    if (stager) {
        c_next = *reinterpret_cast<const float4*>(cblk + (size_t)s_head * T + s_col);
        stage(0, c_next);
    }
    float bt[TW], gt[TW];
#pragma unroll
    for (int j = 0; j < TW; ++j) {
        bt[j] = b_rows[(size_t)j * Dp];
        gt[j] = 0.f;
    }
    // the heads' values, asked for two heads ahead of their use (one ahead leaves the load's
    // latency showing at the end of every head: 170 -> 161 us on the 22.8M-row L1 workload;
    // three ahead measures the same as two)
    float a_q0 = a_rows[0], a_q1 = a_rows[(size_t)min(1, B - 1) * Dp];
    __syncthreads();
    for (int b0 = 0, buf = 0; b0 < B; b0 += L1P_CB, buf ^= 1) {
        const bool more = b0 + L1P_CB < B;
        if (stager && more) c_next = *reinterpret_cast<const float4*>(cblk + (size_t)(b0 + L1P_CB + s_head) * T + s_col);
        if (b0 > 0) {
#pragma unroll
            for (int j4 = 0; j4 < TW; j4 += 4) {
                const float4 h4 = *reinterpret_cast<const float4*>(&col_half[buf ^ 1][l0 + j4]);
                const float hv[4] = {h4.x, h4.y, h4.z, h4.w};
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    if (j4 + x < TW) gt[j4 + x] -= hv[x];
            }
        }
        if (u >= 0) {
            if (u < t_live) {
                float sum = 0.f;
#pragma unroll
                for (int h = 0; h < L1P_CB; ++h) sum += cs[buf][h][u_lds];
                col_half[buf][u_lds] = 0.5f * sum;
            }
            if (u < L1P_CB * L1P_WAVES) {
                const int h = u / L1P_WAVES, v = u % L1P_WAVES;
                float sum = 0.f;
#pragma unroll
                for (int j = 0; j < TW; ++j) sum += cs[buf][h][v * TWS + j];
                row_part[buf][h][v] = sum;
            }
        }
#pragma unroll 1
        for (int bi = 0; bi < L1P_CB; ++bi) {
            const float a = a_q0;
            a_q0 = a_q1;
            a_q1 = a_rows[(size_t)min(b0 + bi + 2, B - 1) * Dp];
            const float* c = &cs[buf][bi][l0];
            float gp = 0.f;
#pragma unroll
            for (int j4 = 0; j4 < TW; j4 += 4) {
                const float4 c4 = *reinterpret_cast<const float4*>(c + j4);
                const float cv[4] = {c4.x, c4.y, c4.z, c4.w};
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    if (j4 + x >= TW) continue;
                    const float p = __builtin_amdgcn_fmed3f(fmaf(a - bt[j4 + x], 0x1p126f, 0.5f), 0.f, 1.f);
                    gp = fmaf(cv[x], p, gp);
                    gt[j4 + x] = fmaf(cv[x], p, gt[j4 + x]);
                }
            }
            part[buf][w][bi][lane] = gp;
        }
        if (stager && more) stage(buf ^ 1, c_next);
        __syncthreads();
        // waves 0 .. 7 add the 16 partials of head b0 + w
        if (w < L1P_CB) {
            float sum = 0.f;
#pragma unroll
            for (int v = 0; v < L1P_WAVES; ++v) sum += fmaf(2.f, part[buf][v][w][lane], -row_part[buf][w][v]);
            grad_a[(size_t)(b0 + w) * Dp] = sum;
        }
    }
    const int last = ((B / L1P_CB) - 1) & 1;
#pragma unroll
    for (int j = 0; j < TW; ++j) grad_b[(size_t)j * Dp] = -2.f * (gt[j] - col_half[last][l0 + j]);
}

__global__ __launch_bounds__(1024) void k_score_bwd_l1_pair(const float* __restrict__ operands,
                                                            const float* __restrict__ coef,
                                                            float* __restrict__ grad, int B, int T,
                                                            int Dp, int a_c0, int b_c0,
                                                            const uint32_t* __restrict__ tcount, int tpad) {
    // the coefficient rows first: their reads in the inner loop then carry the whole address
    // offset in the instruction
    __shared__ __attribute__((aligned(16))) struct {
        float cs[2][L1P_CB][L1P_MAX_T];
        float col_half[2][L1P_MAX_T];
        float row_part[2][L1P_CB][L1P_WAVES];
        float part[2][L1P_WAVES][L1P_CB][64];
    } lds;
    const TileId tile = xcd_tile(Dp / 64, 1, (int)gridDim.x / (Dp / 64));
    const int d = tile.z, lane = threadIdx.x & 63, k = tile.x * 64 + lane;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // merged tails: the block's distinct tails in whole groups of 32 (two per wave), split evenly
    // over the waves.  The columns between that and the forward pass's limit (whole groups of
    // `tpad`) stand for no tail position: their coefficients are zero and nothing reads their
    // gradient rows.  331 instead of 343 columns per block on average on the 22.8M-row workload,
    // and the launch's time follows that average (158.6 -> 155 us), not its largest block.
    const int t_fwd = tail_limit(tcount, d, T, tpad);
    const int t_live = __builtin_amdgcn_readfirstlane(tcount ? min(t_fwd, ((int)tcount[d] + 31) & ~31) : t_fwd);
    const int tw = t_live / L1P_WAVES, t0 = w * tw;
    const float* a_rows = operands + (size_t)(a_c0 + d * B) * Dp + k;
    const float* b_rows = operands + (size_t)(b_c0 + d * T + t0) * Dp + k;
    const float* cblk = coef + (size_t)d * B * T;
    float* grad_a = grad + (size_t)(a_c0 + d * B) * Dp + k;
    float* grad_b = grad + (size_t)(b_c0 + d * T + t0) * Dp + k;
#define KGE_L1P(TW_) \
    case TW_: l1_pair_wave<TW_>(a_rows, b_rows, cblk, grad_a, grad_b, B, T, Dp, t_live, w, lane, lds.part, lds.cs, lds.col_half, lds.row_part); break;
    switch (tw) {  // one of sixteen copies of the loop, chosen per block
        KGE_L1P(2) KGE_L1P(4) KGE_L1P(6) KGE_L1P(8) KGE_L1P(10) KGE_L1P(12) KGE_L1P(14) KGE_L1P(16)
        KGE_L1P(18) KGE_L1P(20) KGE_L1P(22) KGE_L1P(24) KGE_L1P(26) KGE_L1P(28) KGE_L1P(30) KGE_L1P(32)
    }
#undef KGE_L1P
}

// shapes the paired L1 kernel takes: tails split evenly over 16 waves, whole
// chunks of heads, whole 64-column slices, and enough workgroups for the chip
static bool l1_pair_ok(const ScoreShape& sh) {
    // (T % 64 == 0: every live count is a multiple of 32, 2 tails per wave at least)
    return sh.T % 64 == 0 && sh.T >= 128 && sh.T <= L1P_MAX_T && sh.B % L1P_CB == 0 &&
           sh.Dp % 64 == 0 && sh.S * (sh.Dp / 64) >= 128 && (!sh.tcount || sh.tpad == 64);
}

void launch_score_bwd(const ScoreShape& sh, const RowSource& ent, const float* rel,
                      const uint32_t* crel, const float* coef, const uint32_t* nearflag, float* grad,
                      hipStream_t stream) {
    BwdParams p;
    p.ent_a = ent; p.ent_b = ent; p.rel = rel; p.crel = crel; p.coef = coef; p.grad = grad;
    p.coef_div = nullptr; p.add_base = nullptr;
    p.S = sh.S; p.B = sh.B; p.T = sh.T; p.Dp = sh.Dp; p.vec_out = 1; p.use_mfma = sh.use_mfma;
    p.nearflag = nearflag;
    p.tcount = sh.tcount; p.tpad = sh.tpad;
    p.a_rel_mode = sh.operands_dense ? 0 : (sh.score_fn == SCORE_DISTMULT ? 2 : 1);
    p.a_c0 = 0; p.b_c0 = sh.S * sh.B;
    const int dist_fn = sh.score_fn == SCORE_DISTMULT ? DIST_DOT : sh.dist_fn;
    // matrix-core path: both sides in one launch (tile-aligned shapes)
    const bool plain = ent.etype == ET_F32 && !ent.index && p.a_rel_mode == 0 && ent.vec;
    const bool both = sh.use_mfma && plain && sh.B % BM_TI == 0 && sh.T % BM_TI == 0 && sh.Dp % BM_TK == 0 &&
                      (dist_fn == DIST_DOT || (dist_fn == DIST_L2 && nearflag));
    if (both) {
        const dim3 grid = tile_grid(sh.Dp / BM_TK, sh.B / BM_TI + sh.T / BM_TI, sh.S);
        // eight waves per workgroup (two per SIMD): measured faster than four at
        // every benchmark shape, few workgroups (1M-row workload) or many (22.8M-row workload)
        // three-piece bfloat16 products where the forward pass uses them; whole slabs of 32 rows
        // of `other` on either side (the merged tails' live counts are multiples of tpad)
        const bool split = sh.use_mfma == 2 && (!sh.tcount || sh.tpad % (2 * BS_KJ) == 0);
        if (split && dist_fn == DIST_L2)
            hipLaunchKernelGGL(k_score_bwd_split_both<DIST_L2>, grid, dim3(512), 0, stream, p);
        else if (split)
            hipLaunchKernelGGL(k_score_bwd_split_both<DIST_DOT>, grid, dim3(512), 0, stream, p);
        else if (dist_fn == DIST_L2)
            hipLaunchKernelGGL((k_score_bwd_mfma_both<DIST_L2, 32, true, 8>), grid, dim3(512), 0, stream, p);
        else
            hipLaunchKernelGGL((k_score_bwd_mfma_both<DIST_DOT, 32, true, 8>), grid, dim3(512), 0, stream, p);
        return;
    }
    if (dist_fn == DIST_L1 && sh.use_mfma && sh.operands_dense && plain && ent.pitch == (int64_t)sh.Dp * 4 && l1_pair_ok(sh)) {
        const float* ops = reinterpret_cast<const float*>(ent.base);
        const dim3 grid = tile_grid(sh.Dp / 64, 1, sh.S);
        hipLaunchKernelGGL(k_score_bwd_l1_pair, grid, dim3(1024), 0, stream, ops, coef, grad, sh.B, sh.T, sh.Dp, p.a_c0,
                           p.b_c0, sh.tcount, sh.tpad);
        return;
    }
    p.side_b = 0; p.grad_c0 = p.a_c0;
    launch_bwd(p, dist_fn, stream);
    p.side_b = 1; p.grad_c0 = p.b_c0;
    launch_bwd(p, dist_fn, stream);
}


static RowSource plain_rows_bwd(const float* ptr, int D) {
    RowSource s;
    s.base = reinterpret_cast<const char*>(ptr); s.pitch = (int64_t)D * 4; s.etype = ET_F32; s.index = nullptr;
    s.count = D; s.vec = (D % 4 == 0) && ((uintptr_t)ptr % 16 == 0);
    return s;
}

// g [M, N]; dist [M, N] (L2 only, else null): gradient of the first operand
void launch_distance_grad(int dist_fn, const float* a, const float* b, const float* dist,
                          const float* g, float* grad, int M, int N, int D, hipStream_t stream) {
    BwdParams p;
    p.ent_a = plain_rows_bwd(a, D); p.ent_b = plain_rows_bwd(b, D);
    p.rel = nullptr; p.crel = nullptr;
    p.coef = g;
    p.coef_div = dist_fn == DIST_L2 ? dist : nullptr;
    p.grad = grad;
    p.S = 1; p.B = M; p.T = N; p.Dp = D;
    p.side_b = 0; p.a_rel_mode = 0;
    p.a_c0 = 0; p.b_c0 = 0; p.grad_c0 = 0; p.use_mfma = 1; p.nearflag = nullptr;
    p.tcount = nullptr; p.tpad = 1;
    p.vec_out = (D % 4 == 0) && ((uintptr_t)grad % 16 == 0);
    launch_bwd(p, dist_fn, stream);
}

}  // namespace kge
