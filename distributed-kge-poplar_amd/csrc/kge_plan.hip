// gfx950 kernels of the plan phase: the index-only work of a training step, batched over the
// steps of one call.
//
//   merge_tails     a block's tail list reduced to its distinct rows, with multiplicities
//   build_items     every head / tail contribution resolved to its table row
//                   (remote[src][slot], the all-to-all folded into the index arithmetic,
//                   tests/python/reference_model.py:132-138)
//   radix sort      (row, contribution or not, item) order: equal rows adjacent, a row's gradient
//                   contributions in front of its other members, each group ordered by item number
//   find_segments   distinct rows, their members, the chunks of rows with many contributions
//
// Together the device-side counterpart of the host's np.unique (unique_pad,
// src/python/poplar_kge_dataset.py:161-164) and of the grouping multiUpdateAdd does for
// duplicate indices (src/pag/pag.cpp:721-743).  Integer work throughout: every result is exact
// and independent of scheduling (the only atomics are integer counters).
#include "kge_kernels.h"

#include <algorithm>
#include <cstdint>

namespace kge {

#define DEVINL __device__ __forceinline__

// One workgroup per sort tile (kSortTile items) of the entity items or of the relation items of
// one step: the items' keys and values, the per-contribution arrays the step kernels read, and
// the tile's digit histogram for the first radix pass (hist layout as k_sort_hist writes it).
constexpr int kBuildThreads = 1024;
__global__ __launch_bounds__(kBuildThreads) void k_build_items(PlanShape ps, const uint32_t* __restrict__ remote,
                                                     const uint32_t* __restrict__ a2a,
                                                     const uint32_t* __restrict__ head,
                                                     const uint32_t* __restrict__ relation,
                                                     const uint32_t* __restrict__ tail,
                                                     const uint32_t* __restrict__ tkey,
                                                     const uint32_t* __restrict__ tcol,
                                                     uint32_t* __restrict__ ckey,
                                                     uint32_t* __restrict__ crel,
                                                     uint32_t* __restrict__ clabel,
                                                     uint32_t* __restrict__ ent_keys,
                                                     uint32_t* __restrict__ ent_vals,
                                                     uint32_t* __restrict__ rel_keys,
                                                     uint32_t* __restrict__ rel_vals,
                                                     int digit_bits, uint32_t* __restrict__ ent_hist,
                                                     uint32_t* __restrict__ rel_hist) {
    __shared__ uint32_t h[1 << kSortMaxBits];
    const int seg = blockIdx.y, step = ps.step0 + seg, tid = threadIdx.x;
    const int S = ps.S, B = ps.B, A = ps.A, NR = ps.NR, T = S * A;
    const size_t W = (size_t)ps.idx_step_stride;
    const int R = S * NR, SB = S * B;
    const int SBr = SB * ps.rel_copies;
    const int n_rel_items = SBr + ps.n_relation * ps.rel_copies;
    const int e_tiles = (2 * R + kSortTile - 1) / kSortTile, r_tiles = (n_rel_items + kSortTile - 1) / kSortTile;
    const int DIG = 1 << digit_bits;
    const bool entity = (int)blockIdx.x < e_tiles;
    const int tile = entity ? blockIdx.x : blockIdx.x - e_tiles;
    for (int d = tid; d < DIG; d += kBuildThreads) h[d] = 0;
    __syncthreads();
    constexpr int PER = kSortTile / kBuildThreads;  // items per thread; their loads go out together
    if (entity) {
        int item[PER], src[PER];
        uint32_t slot[PER], key[PER];
        const bool merged = ps.merge_tails != 0;
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            item[r] = tile * kSortTile + r * kBuildThreads + tid;
            const int it = item[r];
            slot[r] = 0; src[r] = 0;
            if (it < SB) {
                const int d = it / B, b = it - d * B;
                src[r] = d;
                slot[r] = head[(size_t)step * W + d * B + b];
            } else if (it < R) {
                const int cc = it - SB;
                if (merged) {
                    slot[r] = tkey[(size_t)step * S * T + cc];  // the finished key of the block's column
                } else {
                    const int d = cc / T, t = cc - d * T;
                    const int j = t / A, i = t - j * A;
                    src[r] = j;
                    slot[r] = a2a[(size_t)step * W + ((size_t)j * S + d) * A + i];
                }
            } else if (it < 2 * R) {
                const int sl = it - R;
                src[r] = sl / NR;
                slot[r] = sl - src[r] * NR;
            }
        }
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const uint32_t base = ps.shared_table ? 0u : (uint32_t)src[r] * (uint32_t)ps.n_entity;
            const int it = item[r];
            if (merged && it >= SB && it < R) key[r] = slot[r];
            else if (it < 2 * R)
                key[r] = ((base + remote[(size_t)step * W + (size_t)src[r] * NR + slot[r]]) << kKeyFlagBits) | (it < R ? 0u : 1u);
            else key[r] = 0u;
        }
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            if (item[r] >= 2 * R) continue;
            if (item[r] < R) ckey[(size_t)step * R + item[r]] = key[r] >> kKeyFlagBits;
            ent_keys[(size_t)step * 2 * R + item[r]] = key[r];
            ent_vals[(size_t)step * 2 * R + item[r]] = item[r];
            atomicAdd(&h[key[r] & (uint32_t)(DIG - 1)], 1u);
        }
    } else {
        int item[PER];
        uint32_t key[PER], label[PER];
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            item[r] = tile * kSortTile + r * kBuildThreads + tid;
            const int it = item[r];
            key[r] = 0; label[r] = 0;
            if (it < SBr) {
                const int copy = it / SB, c = it - copy * SB;
                const int d = c / B, b = c - d * B;
                key[r] = relation[(size_t)step * W + d * B + b];
                if (copy == 0) label[r] = tail[(size_t)step * W + d * B + b];
                if (copy == 0 && ps.merge_tails) label[r] = tcol[((size_t)step * S + d) * T + label[r]];
            } else if (it < n_rel_items) {
                key[r] = it - SBr;
            }
        }
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int it = item[r];
            if (it >= n_rel_items) continue;
            uint32_t k = key[r];
            if (it < SBr) {
                const int copy = it / SB, c = it - copy * SB;
                if (copy == 0) {
                    crel[(size_t)step * SB + c] = k;
                    clabel[(size_t)step * SB + c] = label[r];
                }
                k += (uint32_t)(copy * ps.n_relation);
            }
            k = (k << kKeyFlagBits) | (it < SBr ? 0u : 1u);
            rel_keys[(size_t)step * n_rel_items + it] = k;
            rel_vals[(size_t)step * n_rel_items + it] = it;
            atomicAdd(&h[k & (uint32_t)(DIG - 1)], 1u);
        }
    }
    __syncthreads();
    uint32_t* hrow = (entity ? ent_hist : rel_hist) + ((size_t)seg * ((entity ? e_tiles : r_tiles) + 1) + tile) * DIG;
    for (int d = tid; d < DIG; d += kBuildThreads) hrow[d] = h[d];
}

void launch_build_items(const PlanShape& ps, const uint32_t* remote, const uint32_t* a2a,
                        const uint32_t* head, const uint32_t* relation, const uint32_t* tail,
                        const uint32_t* tkey, const uint32_t* tcol,
                        uint32_t* ckey, uint32_t* crel, uint32_t* clabel, uint32_t* ent_keys,
                        uint32_t* ent_vals, uint32_t* rel_keys, uint32_t* rel_vals, int digit_bits,
                        uint32_t* ent_hist, uint32_t* rel_hist, hipStream_t stream) {
    const int R = ps.S * ps.NR, n_rel_items = (ps.S * ps.B + ps.n_relation) * ps.rel_copies;
    const int e_tiles = (2 * R + kSortTile - 1) / kSortTile, r_tiles = (n_rel_items + kSortTile - 1) / kSortTile;
    dim3 grid(e_tiles + r_tiles, ps.step_count);
    hipLaunchKernelGGL(k_build_items, grid, dim3(kBuildThreads), 0, stream, ps, remote, a2a, head, relation,
                       tail, tkey, tcol, ckey, crel, clabel, ent_keys, ent_vals, rel_keys, rel_vals, digit_bits, ent_hist,
                       rel_hist);
}

// items for a plain scatter-add: n real items keyed by idx, then one
// zero-gradient item per table row so that every row forms a segment
__global__ __launch_bounds__(256) void k_iota_keys(const uint32_t* __restrict__ idx,
                                                   uint32_t* __restrict__ keys,
                                                   uint32_t* __restrict__ vals, int64_t n,
                                                   int64_t rows) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n + rows) return;
    // an index outside the table carries no gradient anywhere: it joins row 0's other members
    const uint32_t row = i < n ? idx[i] : (uint32_t)(i - n);
    const bool real = i < n && (int64_t)row < rows;
    keys[i] = ((real || i >= n ? row : 0u) << kKeyFlagBits) | (real ? 0u : 1u);
    vals[i] = (uint32_t)i;
}
void launch_iota_keys(const uint32_t* idx, uint32_t* keys, uint32_t* vals, int64_t n, int64_t rows,
                      hipStream_t stream) {
    hipLaunchKernelGGL(k_iota_keys, dim3((unsigned)((n + rows + 255) / 256)), dim3(256), 0, stream, idx, keys, vals,
                       n, rows);
}

// ---- stable LSD radix sort -------------------------------------------------------------------
// As few passes as the key width allows with digits of at most 11 bits (20-bit row numbers: two
// passes of 10; 25 bits: 9 + 8 + 8; a relation table's 11 bits: one pass).  Two launches per
// pass (the first pass's histograms come from k_build_items; the entity and the relation sort
// of a training call share their launches): tile histograms, then the stable scatter, whose workgroups each derive their output
// positions from the histograms of all tiles (one round of loads; a separate scan launch, or
// workgroups that hand results to each other through fences, both cost more than the reads).
// hist layout: [seg][tile][digit] (digits contiguous: every access below is coalesced), n_tiles + 1
// rows per segment.  Arrays of more than kSortFoldTiles tiles (the stand-alone scatter-add on
// millions of items; a training call's arrays have a few dozen) get a scan launch between the two:
// every tile's row then holds the counts of the tiles in front of it and row n_tiles the totals,
// so that a scatter workgroup reads two rows instead of all of them.

SortPasses sort_passes(int key_bits) {
    SortPasses p = {};
    key_bits = std::max(1, key_bits);
    p.n = (key_bits + kSortMaxBits - 1) / kSortMaxBits;
    const int base = key_bits / p.n, extra = key_bits % p.n;
    int shift = 0;
    for (int i = 0; i < p.n; ++i) {
        p.bits[i] = base + (i < extra ? 1 : 0);
        p.shift[i] = shift;
        shift += p.bits[i];
    }
    return p;
}

size_t radix_sort_hist_words(int N, int n_seg, int key_bits) {
    const SortPasses p = sort_passes(key_bits);
    const size_t n_tiles = ((size_t)N + kSortTile - 1) / kSortTile;
    // the first pass has the widest digit; one more row per segment for the digit totals of a scanned histogram
    return (size_t)n_seg * ((size_t)1 << p.bits[0]) * (n_tiles + 1);
}

// Which of a launch's two jobs a workgroup serves: blockIdx.x counts job 0's tiles, then job 1's.
DEVINL const SortJob& sort_job(const SortJob& j0, const SortJob& j1, int& tile) {
    tile = blockIdx.x;
    if (tile < j0.n_tiles) return j0;
    tile -= j0.n_tiles;
    return j1;
}

template <int BITS>
__global__ __launch_bounds__(256) void k_sort_hist(SortJob j0, SortJob j1, int shift) {
    constexpr int DIG = 1 << BITS;
    __shared__ uint32_t h[DIG];
    int tile;
    const SortJob& job = sort_job(j0, j1, tile);
    const int seg = blockIdx.y, tid = threadIdx.x, N = job.N;
    const uint32_t* __restrict__ k = job.keys_in + (size_t)seg * N;
    const int base = tile * kSortTile;
    uint32_t key[kSortTile / 256];
#pragma unroll
    for (int r = 0; r < kSortTile / 256; ++r) {
        const int i = base + r * 256 + tid;
        key[r] = i < N ? k[i] : 0u;
    }
    for (int d = tid; d < DIG; d += 256) h[d] = 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortTile / 256; ++r)
        if (base + r * 256 + tid < N) atomicAdd(&h[(key[r] >> shift) & (DIG - 1)], 1u);
    __syncthreads();
    uint32_t* hrow = job.hist + ((size_t)seg * (job.n_tiles + 1) + tile) * DIG;
    for (int d = tid; d < DIG; d += 256) hrow[d] = h[d];
}

constexpr int kSortFoldTiles = 64;
// one thread per (segment, digit): the tiles' counts become exclusive prefixes over the tiles,
// row n_tiles the totals
template <int BITS>
__global__ __launch_bounds__(256) void k_sort_scan(SortJob job) {
    constexpr int DIG = 1 << BITS;
    const int d = blockIdx.x * 256 + threadIdx.x, seg = blockIdx.y;
    if (d >= DIG) return;
    uint32_t* h = job.hist + (size_t)seg * (job.n_tiles + 1) * DIG + d;
    uint32_t run = 0;
    int t = 0;
    for (; t + 8 <= job.n_tiles; t += 8) {  // eight loads in flight
        uint32_t c[8];
#pragma unroll
        for (int x = 0; x < 8; ++x) c[x] = h[(size_t)(t + x) * DIG];
#pragma unroll
        for (int x = 0; x < 8; ++x) { h[(size_t)(t + x) * DIG] = run; run += c[x]; }
    }
    for (; t < job.n_tiles; ++t) { const uint32_t c = h[(size_t)t * DIG]; h[(size_t)t * DIG] = run; run += c; }
    h[(size_t)job.n_tiles * DIG] = run;
}

template <int BITS>
__global__ __launch_bounds__(256) void k_sort_scatter(SortJob j0, SortJob j1, int shift) {
    constexpr int DIG = 1 << BITS;
    constexpr int DPT = (DIG + 255) / 256;  // digits per thread
    // run[w][digit]: next output position for wave w's items with that digit
    __shared__ uint32_t run[4][DIG];
    __shared__ uint32_t s_tot[DPT * 256];   // items of each digit in all tiles, then their exclusive prefix
    __shared__ uint32_t wtot[4];
    int tile;
    const SortJob& job = sort_job(j0, j1, tile);
    const int seg = blockIdx.y, N = job.N, n_tiles = job.n_tiles;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const uint32_t* __restrict__ kin = job.keys_in + (size_t)seg * N;
    const uint32_t* __restrict__ vin = job.vals_in + (size_t)seg * N;
    const uint32_t* __restrict__ hist = job.hist;
    constexpr int ROUNDS = kSortTile / 256;  // rounds of 64 items per wave
    const int wbase = tile * kSortTile + wave * (kSortTile / 4);

    uint32_t key[ROUNDS], val[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const int i = wbase + r * 64 + lane;
        key[r] = i < N ? kin[i] : 0xffffffffu;
        val[r] = i < N ? vin[i] : 0u;
    }
    // This tile's first output position of every digit, from the histograms of all tiles: items
    // of smaller digits anywhere, then items of the same digit in earlier tiles.
    // Step 1: thread t sums digits t, t + 256, ... over the tiles (lanes read consecutive words).
    uint32_t pre[DPT];
    {
        const uint32_t* hseg = hist + (size_t)seg * (n_tiles + 1) * DIG;
        uint32_t tot[DPT];
#pragma unroll
        for (int q = 0; q < DPT; ++q) { tot[q] = 0; pre[q] = 0; }
        if (n_tiles > kSortFoldTiles) {  // scanned by k_sort_scan
#pragma unroll
            for (int q = 0; q < DPT; ++q) {
                const int d = q * 256 + tid;
                pre[q] = d < DIG ? hseg[(size_t)tile * DIG + d] : 0u;
                tot[q] = d < DIG ? hseg[(size_t)n_tiles * DIG + d] : 0u;
            }
        } else
        for (int t0 = 0; t0 < n_tiles; t0 += 8) {  // eight tiles' rows in flight: one round trip per eight tiles
            uint32_t c[8][DPT];
#pragma unroll
            for (int x = 0; x < 8; ++x)
#pragma unroll
                for (int q = 0; q < DPT; ++q) {
                    const int d = q * 256 + tid;
                    c[x][q] = (t0 + x < n_tiles && d < DIG) ? hseg[(size_t)(t0 + x) * DIG + d] : 0u;
                }
#pragma unroll
            for (int x = 0; x < 8; ++x)
#pragma unroll
                for (int q = 0; q < DPT; ++q) {
                    tot[q] += c[x][q];
                    pre[q] += t0 + x < tile ? c[x][q] : 0u;
                }
        }
#pragma unroll
        for (int q = 0; q < DPT; ++q) s_tot[q * 256 + tid] = tot[q];
    }
    for (int i = tid; i < 4 * DIG; i += 256) (&run[0][0])[i] = 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r)
        if (wbase + r * 64 + lane < N) atomicAdd(&run[wave][(key[r] >> shift) & (DIG - 1)], 1u);
    {   // step 2: exclusive scan of the digit totals; thread t owns digits [t * DPT, (t + 1) * DPT)
        uint32_t mine[DPT], sum = 0;
#pragma unroll
        for (int q = 0; q < DPT; ++q) { mine[q] = s_tot[tid * DPT + q]; sum += mine[q]; }
        uint32_t inc = sum;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const uint32_t t = __shfl_up(inc, off, 64);
            if (lane >= off) inc += t;
        }
        if (lane == 63) wtot[wave] = inc;
        __syncthreads();  // also: every thread has read its s_tot entries, every wave's counts are in run[][]
        uint32_t base = inc - sum;
#pragma unroll
        for (int w = 0; w < 4; ++w) base += w < wave ? wtot[w] : 0u;
#pragma unroll
        for (int q = 0; q < DPT; ++q) {
            s_tot[tid * DPT + q] = base;
            base += mine[q];
        }
    }
    __syncthreads();
    // step 3: per digit the exclusive prefix over the four waves on top of the tile's base
#pragma unroll
    for (int q = 0; q < DPT; ++q) {
        const int d = q * 256 + tid;
        if (d < DIG) {
            uint32_t b = s_tot[d] + pre[q];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t c = run[w][d];
                run[w][d] = b;
                b += c;
            }
        }
    }
    __syncthreads();
    uint32_t* __restrict__ kout = job.keys_out + (size_t)seg * N;
    uint32_t* __restrict__ vout = job.vals_out + (size_t)seg * N;
    // a wave's counters are its own: the rounds need no workgroup barrier, only the order of
    // the wave's own LDS accesses
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const int i = wbase + r * 64 + lane;
        const bool valid = i < N;
        const uint32_t digit = (key[r] >> shift) & (DIG - 1);
        // lanes of this wave holding the same digit (match-any by BITS ballots)
        uint64_t peers = __ballot(valid);
#pragma unroll
        for (int bit = 0; bit < BITS; ++bit) {
            const uint64_t m = __ballot((digit >> bit) & 1u);
            peers &= ((digit >> bit) & 1u) ? m : ~m;
        }
        const uint64_t lt = (1ull << lane) - 1ull;
        const uint32_t rank = __popcll(peers & lt);
        uint32_t off = 0;
        if (valid) off = run[wave][digit];
        __builtin_amdgcn_wave_barrier();
        if (valid && rank == 0) run[wave][digit] = off + (uint32_t)__popcll(peers);
        __builtin_amdgcn_wave_barrier();
        if (valid) {
            kout[off + rank] = key[r];
            vout[off + rank] = val[r];
        }
    }
}

// Two sorts in shared launches.  The pass schedule is that of the wider key; a job takes part in
// the passes that still cover bits of its own keys (a prefix of them) and ends in its b buffers
// after an odd number of passes.  `first_hist_done`: the caller has already written both jobs'
// histograms of pass 0 (k_build_items).  j1 may be null.
void launch_radix_sort2(SortBuffers* j0, SortBuffers* j1, int n_seg, bool first_hist_done, hipStream_t stream) {
    const SortPasses sp = sort_passes(std::max(j0->key_bits, j1 ? j1->key_bits : 1));
    SortBuffers* jobs[2] = {j0, j1};
    SortJob cur[2] = {};
    for (int q = 0; q < 2; ++q) {
        if (!jobs[q]) continue;
        cur[q].keys_in = jobs[q]->keys_a; cur[q].vals_in = jobs[q]->vals_a;
        cur[q].keys_out = jobs[q]->keys_b; cur[q].vals_out = jobs[q]->vals_b;
        cur[q].hist = jobs[q]->hist; cur[q].N = jobs[q]->N;
        cur[q].n_tiles = (jobs[q]->N + kSortTile - 1) / kSortTile;
        jobs[q]->result_in_b = 0;
    }
    for (int p = 0; p < sp.n; ++p) {
        const int shift = sp.shift[p];
        SortJob a[2] = {};
        int n = 0;
        for (int q = 0; q < 2; ++q)
            if (jobs[q] && (p == 0 || shift < jobs[q]->key_bits)) a[n++] = cur[q];
        if (n == 0) break;
        if (n == 1) a[1].n_tiles = 0;
        const dim3 grid(a[0].n_tiles + a[1].n_tiles, n_seg);
        const bool hist_done = p == 0 && first_hist_done;
#define KGE_SORT_PASS(B_)                                                                                     \
    case B_:                                                                                                  \
        if (!hist_done) hipLaunchKernelGGL(k_sort_hist<B_>, grid, dim3(256), 0, stream, a[0], a[1], shift);   \
        for (int q = 0; q < n; ++q)                                                                           \
            if (a[q].n_tiles > kSortFoldTiles)                                                                \
                hipLaunchKernelGGL(k_sort_scan<B_>, dim3(((1 << B_) + 255) / 256, n_seg), dim3(256), 0, stream, a[q]); \
        hipLaunchKernelGGL(k_sort_scatter<B_>, grid, dim3(256), 0, stream, a[0], a[1], shift);                \
        break;
        switch (sp.bits[p]) {
            KGE_SORT_PASS(1) KGE_SORT_PASS(2) KGE_SORT_PASS(3) KGE_SORT_PASS(4) KGE_SORT_PASS(5) KGE_SORT_PASS(6)
            KGE_SORT_PASS(7) KGE_SORT_PASS(8) KGE_SORT_PASS(9) KGE_SORT_PASS(10) KGE_SORT_PASS(11)
        }
#undef KGE_SORT_PASS
        for (int q = 0; q < 2; ++q)
            if (jobs[q] && (p == 0 || shift < jobs[q]->key_bits)) {
                std::swap(cur[q].keys_in, cur[q].keys_out);
                std::swap(cur[q].vals_in, cur[q].vals_out);
                jobs[q]->result_in_b ^= 1;
            }
    }
}

int launch_radix_sort(uint32_t* keys_a, uint32_t* vals_a, uint32_t* keys_b, uint32_t* vals_b,
                      uint32_t* hist, int N, int n_seg, int key_bits, hipStream_t stream) {
    SortBuffers j = {};
    j.keys_a = keys_a; j.vals_a = vals_a; j.keys_b = keys_b; j.vals_b = vals_b; j.hist = hist;
    j.N = N; j.key_bits = key_bits;
    launch_radix_sort2(&j, nullptr, n_seg, false, stream);
    return j.result_in_b;
}

// ---- segments and chunks ---------------------------------------------------------------------
// Three launches over tiles of 2048 sorted items (256 threads x 8 consecutive items), both
// plans of every step in each launch, nothing handed between workgroups inside a launch:
//   1. count: row starts per tile (a row starts where the key's row number changes) and the tile's last one
//   2. rows:  with the earlier tiles' counts in front, every item knows its distinct-row index
//      and its row's first position.  Within a row the gradient contributions (key flag 0)
//      come first, and every row holds at least one other member (its `remote` slot / the
//      scatter-add's one item per table row): the first of those knows the row's number of
//      contributions and "owns" the row.
//      The rows a tile owns are consecutive; their chunk counts are summed per tile.
//   3. chunks: with the earlier tiles' chunk counts in front, the chunk tables of rows with more
//      than direct_max contributions and the list of those rows.

constexpr int kSegTile = 2048, kSegPer = 8;
static_assert(kSegTile == 256 * kSegPer, "256 threads x kSegPer items");

// per (array, tile): words of SegScratch::tile_info
//   0 row starts in the tile   1 (position of the tile's last row start) + 1, 0 if none
//   2 chunks of the rows the tile owns   3 how many of them have chunks   4 the most contributions among them
//   5 rows the tile owns   6 the first of them
constexpr int kSegInfo = 8;

// kSegPer consecutive words from p + i0 (words past n read as zero); 16-byte loads when `vec`
DEVINL void load_run(const uint32_t* __restrict__ p, int i0, int n, bool vec, uint32_t out[kSegPer]) {
    if (vec && i0 + kSegPer <= n) {
#pragma unroll
        for (int x = 0; x < kSegPer; x += 4) {
            const uint4 v = *reinterpret_cast<const uint4*>(p + i0 + x);
            out[x] = v.x; out[x + 1] = v.y; out[x + 2] = v.z; out[x + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int x = 0; x < kSegPer; ++x) out[x] = i0 + x < n ? p[i0 + x] : 0u;
    }
}

struct SegWg {  // what every segment kernel derives from its block index
    const SegJob* job;
    int seg, tile, n_tiles, slot;  // slot: index of (job, seg) in the scratch arrays
};
DEVINL bool seg_workgroup(const SegJob& j0, const SegJob& j1, int n_seg, SegWg& w) {
    const int y = blockIdx.y;
    w.job = y >= n_seg ? &j1 : &j0;
    w.seg = y >= n_seg ? y - n_seg : y;
    w.slot = y;
    w.tile = blockIdx.x;
    w.n_tiles = (w.job->N + kSegTile - 1) / kSegTile;
    return w.tile < w.n_tiles;
}

// (sum, max) over the workgroup's 256 threads, to every thread
DEVINL void block_sum_max(uint32_t& a, uint32_t& b, uint32_t (*lds)[2]) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        a += __shfl_xor(a, off, 64);
        b = max(b, __shfl_xor(b, off, 64));
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { lds[wave][0] = a; lds[wave][1] = b; }
    __syncthreads();
    a = lds[0][0] + lds[1][0] + lds[2][0] + lds[3][0];
    b = max(max(lds[0][1], lds[1][1]), max(lds[2][1], lds[3][1]));
    __syncthreads();
}

// exclusive scan of (a: sum, b: sum or maximum) over the workgroup's 256 threads in thread
// order; total: the whole workgroup's
template <bool MAX_B>
DEVINL void block_scan_256(uint32_t a, uint32_t b, uint32_t (*lds)[2], uint32_t& ea, uint32_t& eb,
                           uint32_t& ta, uint32_t& tb) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t ia = a, ib = b;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const uint32_t xa = __shfl_up(ia, off, 64), xb = __shfl_up(ib, off, 64);
        if (lane >= off) { ia += xa; ib = MAX_B ? max(ib, xb) : ib + xb; }
    }
    if (lane == 63) { lds[wave][0] = ia; lds[wave][1] = ib; }
    ea = __shfl_up(ia, 1, 64); eb = __shfl_up(ib, 1, 64);
    if (lane == 0) { ea = 0u; eb = 0u; }
    __syncthreads();
    ta = 0u; tb = 0u;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t ca = lds[w][0], cb = lds[w][1];
        if (w < wave) { ea += ca; eb = MAX_B ? max(eb, cb) : eb + cb; }
        ta += ca; tb = MAX_B ? max(tb, cb) : tb + cb;
    }
    __syncthreads();
}

// the row-start flags of this thread's items (bit x: item i0 + x starts a row)
DEVINL uint32_t start_flags(const uint32_t k[kSegPer], uint32_t k_prev, int i0, int N) {
    uint32_t flags = 0;
#pragma unroll
    for (int x = 0; x < kSegPer; ++x) {
        const int i = i0 + x;
        if (i < N && (i == 0 || (k[x] >> kKeyFlagBits) != ((x ? k[x - 1] : k_prev) >> kKeyFlagBits))) flags |= 1u << x;
    }
    return flags;
}

__global__ __launch_bounds__(256) void k_seg_count(SegJob j0, SegJob j1, int n_seg, int max_tiles,
                                                   uint32_t* __restrict__ tile_info) {
    __shared__ uint32_t lds[4][2];
    SegWg w;
    if (!seg_workgroup(j0, j1, n_seg, w)) return;
    const int N = w.job->N, tid = threadIdx.x;
    const uint32_t* __restrict__ keys = w.job->keys + (size_t)w.seg * N;
    const bool vec = (reinterpret_cast<uintptr_t>(keys) & 15) == 0;
    const int i0 = w.tile * kSegTile + kSegPer * tid;
    uint32_t k[kSegPer];
    load_run(keys, i0, N, vec, k);
    const uint32_t k_prev = (i0 > 0 && i0 < N) ? keys[i0 - 1] : 0u;
    const uint32_t flags = start_flags(k, k_prev, i0, N);
    uint32_t cnt = __popc(flags), mx = flags ? (uint32_t)(i0 + 31 - __clz(flags)) + 1u : 0u;
    block_sum_max(cnt, mx, lds);
    if (tid == 0) {
        uint32_t* info = tile_info + ((size_t)w.slot * max_tiles + w.tile) * kSegInfo;
        info[0] = cnt; info[1] = mx;
    }
}

__global__ __launch_bounds__(256) void k_seg_rows(SegJob j0, SegJob j1, int n_seg, int max_tiles,
                                                  uint32_t* __restrict__ tile_info) {
    __shared__ uint32_t lds[4][2];
    SegWg w;
    if (!seg_workgroup(j0, j1, n_seg, w)) return;
    const SegJob& job = *w.job;
    const int N = job.N, tid = threadIdx.x, seg = w.seg;
    const uint32_t n_real = (uint32_t)job.n_real, chunk = (uint32_t)job.chunk, direct_max = (uint32_t)job.direct_max;
    const SegPlan& plan = job.plan;
    const uint32_t* __restrict__ keys = job.keys + (size_t)seg * N;
    const uint32_t* __restrict__ vals = job.vals + (size_t)seg * N;
    uint32_t* __restrict__ uniq_key = plan.uniq_key + (size_t)seg * plan.u_stride;
    uint32_t* __restrict__ seg_start = plan.seg_start + (size_t)seg * (plan.u_stride + 1);
    uint32_t* __restrict__ item_row = plan.item_row ? plan.item_row + (size_t)seg * n_real : nullptr;
    uint32_t* __restrict__ seg_real = plan.seg_real + (size_t)seg * plan.u_stride;
    uint32_t* info_seg = tile_info + (size_t)w.slot * max_tiles * kSegInfo;

    const bool vec = ((reinterpret_cast<uintptr_t>(keys) | reinterpret_cast<uintptr_t>(vals)) & 15) == 0;
    const int i0 = w.tile * kSegTile + kSegPer * tid;
    uint32_t k[kSegPer], v[kSegPer];
    load_run(keys, i0, N, vec, k);
    load_run(vals, i0, N, vec, v);
    const bool has_prev = i0 > 0 && i0 < N;
    const uint32_t k_prev = has_prev ? keys[i0 - 1] : 0u;
    // the earlier tiles: rows started in them, and the last start among them
    uint32_t rows_before = 0, start1_before = 0;
    for (int t = tid; t < w.tile; t += 256) {
        rows_before += info_seg[(size_t)t * kSegInfo];
        start1_before = max(start1_before, info_seg[(size_t)t * kSegInfo + 1]);
    }
    block_sum_max(rows_before, start1_before, lds);

    const uint32_t flags = start_flags(k, k_prev, i0, N);
    const uint32_t cnt = __popc(flags), mx = flags ? (uint32_t)(i0 + 31 - __clz(flags)) + 1u : 0u;
    uint32_t ea, eb, total_rows, total_mx;
    block_scan_256<true>(cnt, mx, lds, ea, eb, total_rows, total_mx);
    uint32_t u = rows_before + ea;                 // rows started in front of this thread's items
    uint32_t start1 = max(start1_before, eb);      // (first position of the row open there) + 1
    uint32_t own_chunks = 0, own_hot = 0, own_big = 0, own_rows = 0, own_first = 0xffffffffu;
#pragma unroll
    for (int x = 0; x < kSegPer; ++x) {
        const int i = i0 + x;
        if (i < N) {
            const bool f = (flags >> x) & 1u;
            if (f) {
                uniq_key[u] = k[x] >> kKeyFlagBits;
                seg_start[u] = (uint32_t)i;
                start1 = (uint32_t)i + 1u;
                ++u;
            }
            // u - 1 is this item's row, start1 - 1 that row's first position
            if (item_row && v[x] < n_real) item_row[v[x]] = u - 1;
            // the row's first member that is no contribution: its contributions lie in front of it
            if ((k[x] & 1u) && (f || !((x ? k[x - 1] : k_prev) & 1u))) {
                const uint32_t real = (uint32_t)i - (start1 - 1u);
                seg_real[u - 1] = real;
                const uint32_t nch = real > direct_max ? (real + chunk - 1) / chunk : 0u;
                own_chunks += nch; own_hot += nch ? 1u : 0u; own_big = max(own_big, real);
                own_first = min(own_first, u - 1); ++own_rows;
            }
        }
    }
    block_sum_max(own_chunks, own_big, lds);
    uint32_t not_first = ~own_first;   // minimum through the maximum
    block_sum_max(own_hot, not_first, lds);
    uint32_t zero = 0;
    block_sum_max(own_rows, zero, lds);
    if (tid == 0) {
        uint32_t* info = info_seg + (size_t)w.tile * kSegInfo;
        info[2] = own_chunks; info[3] = own_hot; info[4] = own_big; info[5] = own_rows; info[6] = ~not_first;
        if (w.tile == w.n_tiles - 1) {
            const uint32_t U = rows_before + total_rows;
            seg_start[U] = (uint32_t)N;
            plan.counts[2 * seg] = U;
            if (plan.host_counts) plan.host_counts[4 * (size_t)seg] = U;
        }
    }
}

__global__ __launch_bounds__(256) void k_seg_chunks(SegJob j0, SegJob j1, int n_seg, int max_tiles,
                                                    const uint32_t* __restrict__ tile_info) {
    __shared__ uint32_t lds[4][2];
    SegWg w;
    if (!seg_workgroup(j0, j1, n_seg, w)) return;
    const SegJob& job = *w.job;
    const int tid = threadIdx.x, seg = w.seg;
    const uint32_t chunk = (uint32_t)job.chunk, direct_max = (uint32_t)job.direct_max;
    const SegPlan& plan = job.plan;
    const uint32_t* __restrict__ seg_start = plan.seg_start + (size_t)seg * (plan.u_stride + 1);
    const uint32_t* __restrict__ seg_real = plan.seg_real + (size_t)seg * plan.u_stride;
    uint32_t* __restrict__ chunk_off = plan.chunk_off + (size_t)seg * (plan.u_stride + 1);
    uint32_t* __restrict__ chunk_pos = plan.chunk_pos + (size_t)seg * plan.c_stride;
    uint32_t* __restrict__ chunk_len = plan.chunk_len + (size_t)seg * plan.c_stride;
    uint32_t* __restrict__ hot = plan.hot_rows ? plan.hot_rows + (size_t)seg * plan.c_stride : nullptr;
    uint32_t* __restrict__ crow = plan.chunk_row ? plan.chunk_row + (size_t)seg * plan.c_stride : nullptr;
    const uint32_t* info_seg = tile_info + (size_t)w.slot * max_tiles * kSegInfo;

    // chunks and rows with chunks that the earlier tiles own
    uint32_t chunks_before = 0, hot_before = 0;
    for (int t = tid; t < w.tile; t += 256) {
        chunks_before += info_seg[(size_t)t * kSegInfo + 2];
        hot_before += info_seg[(size_t)t * kSegInfo + 3];
    }
    {
        uint32_t z0 = 0, z1 = 0;
        block_sum_max(chunks_before, z0, lds);
        block_sum_max(hot_before, z1, lds);
    }
    const uint32_t* info = info_seg + (size_t)w.tile * kSegInfo;
    const uint32_t own_rows = info[5], own_first = info[6];
    // the rows this tile owns are consecutive: kSegPer of them per thread, in order
    uint32_t real[kSegPer], nch[kSegPer], mine = 0, hot_mine = 0;
    const uint32_t r0 = (uint32_t)(kSegPer * tid);
#pragma unroll
    for (int x = 0; x < kSegPer; ++x) {
        real[x] = r0 + x < own_rows ? seg_real[own_first + r0 + x] : 0u;
        nch[x] = real[x] > direct_max ? (real[x] + chunk - 1) / chunk : 0u;
        mine += nch[x];
        hot_mine += nch[x] ? 1u : 0u;
    }
    uint32_t ea, eb, ta, tb;
    block_scan_256<false>(mine, hot_mine, lds, ea, eb, ta, tb);
    uint32_t cb = chunks_before + ea, hb = hot_before + eb;
#pragma unroll
    for (int x = 0; x < kSegPer; ++x) {
        if (r0 + x < own_rows) {
            const uint32_t u = own_first + r0 + x;
            chunk_off[u] = cb;
            if (nch[x]) {
                const uint32_t s = seg_start[u];
                for (uint32_t l = 0; l < nch[x]; ++l) {
                    chunk_pos[cb + l] = s + l * chunk;
                    chunk_len[cb + l] = min(chunk, real[x] - l * chunk);
                    if (crow) crow[cb + l] = u;
                }
                cb += nch[x];
                if (hot) hot[hb] = u;
                ++hb;
            }
        }
    }
    if (w.tile == w.n_tiles - 1) {  // the totals, by the workgroup that has every tile in front of it
        uint32_t biggest = 0, z = 0;
        for (int t = tid; t < w.n_tiles; t += 256) biggest = max(biggest, info_seg[(size_t)t * kSegInfo + 4]);
        block_sum_max(z, biggest, lds);
        if (tid == 0) {
            const uint32_t U = plan.counts[2 * seg], NC = chunks_before + ta, H = hot_before + tb;
            chunk_off[U] = NC;
            plan.counts[2 * seg + 1] = NC;
            if (plan.hot_count) { plan.hot_count[2 * seg] = H; plan.hot_count[2 * seg + 1] = biggest; }
            if (plan.host_counts) {
                uint32_t* h = plan.host_counts + 4 * (size_t)seg;
                h[1] = NC; h[2] = H; h[3] = biggest;
            }
        }
    }
}

size_t find_segments_scratch_words(int N0, int N1, int n_seg) {
    const size_t max_tiles = ((size_t)std::max(N0, N1) + kSegTile - 1) / kSegTile;
    return 2 * (size_t)n_seg * max_tiles * kSegInfo;
}

void launch_find_segments2(const SegJob& j0, const SegJob* j1, int n_seg, uint32_t* scratch, hipStream_t stream) {
    const SegJob& second = j1 ? *j1 : j0;
    const int max_tiles = (std::max(j0.N, j1 ? j1->N : 0) + kSegTile - 1) / kSegTile;
    const dim3 grid(max_tiles, j1 ? 2 * n_seg : n_seg);
    hipLaunchKernelGGL(k_seg_count, grid, dim3(256), 0, stream, j0, second, n_seg, max_tiles, scratch);
    hipLaunchKernelGGL(k_seg_rows, grid, dim3(256), 0, stream, j0, second, n_seg, max_tiles, scratch);
    hipLaunchKernelGGL(k_seg_chunks, grid, dim3(256), 0, stream, j0, second, n_seg, max_tiles, scratch);
}

// ---- merged tails ----------------------------------------------------------------------------
// One workgroup per (block, step): the block's T tail rows (resolved like the tail contributions
// in k_build_items) are sorted together with their positions by a bitonic network in LDS; a
// distinct row becomes a column, numbered in ascending row order.
constexpr int kMergeThreads = 256;
__global__ __launch_bounds__(kMergeThreads) void k_merge_tails(PlanShape ps, const uint32_t* __restrict__ remote,
                                                               const uint32_t* __restrict__ a2a,
                                                               uint32_t* __restrict__ tkey, float* __restrict__ tmult,
                                                               uint32_t* __restrict__ tcol,
                                                               uint32_t* __restrict__ tcount) {
    __shared__ uint64_t e[kMergeMaxT];          // (row, position), ascending after the sort
    __shared__ uint32_t first[kMergeMaxT + 1];  // sorted index of every column's first entry
    __shared__ uint32_t lds[4][2];
    const int d = blockIdx.x, seg = blockIdx.y, step = ps.step0 + seg, tid = threadIdx.x;
    const int S = ps.S, A = ps.A, NR = ps.NR, T = S * A;
    const size_t W = (size_t)ps.idx_step_stride;
    int N = 1;
    while (N < T) N <<= 1;
    for (int i = tid; i < N; i += kMergeThreads) {
        uint64_t v = ~0ull;  // padding sorts behind every row
        if (i < T) {
            const int j = i / A, ii = i - j * A;
            const uint32_t slot = a2a[(size_t)step * W + ((size_t)j * S + d) * A + ii];
            const uint32_t base = ps.shared_table ? 0u : (uint32_t)j * (uint32_t)ps.n_entity;
            const uint32_t row = base + remote[(size_t)step * W + (size_t)j * NR + slot];
            v = ((uint64_t)row << 32) | (uint32_t)i;
        }
        e[i] = v;
    }
    __syncthreads();
    for (int k = 2; k <= N; k <<= 1)
        for (int j = k >> 1; j > 0; j >>= 1) {
            for (int i = tid; i < N / 2; i += kMergeThreads) {
                const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1)), hi = lo | j;
                const uint64_t a = e[lo], b = e[hi];
                if ((a > b) == ((lo & k) == 0)) { e[lo] = b; e[hi] = a; }
            }
            __syncthreads();
        }
    // thread t owns sorted entries [t * per, (t + 1) * per)
    const int per = (N + kMergeThreads - 1) / kMergeThreads;
    const int i0 = tid * per;
    uint32_t mine = 0;
    for (int x = 0; x < per; ++x) {
        const int i = i0 + x;
        if (i < T && (i == 0 || (uint32_t)(e[i] >> 32) != (uint32_t)(e[i - 1] >> 32))) ++mine;
    }
    uint32_t before, eb, total, tb;
    block_scan_256<false>(mine, 0u, lds, before, eb, total, tb);
    const size_t out = ((size_t)step * S + d) * T;
    uint32_t col = before;  // columns started in front of this thread's entries
    for (int x = 0; x < per; ++x) {
        const int i = i0 + x;
        if (i >= T) break;
        const uint32_t row = (uint32_t)(e[i] >> 32), pos = (uint32_t)e[i];
        if (i == 0 || row != (uint32_t)(e[i - 1] >> 32)) {
            first[col] = (uint32_t)i;
            tkey[out + col] = row << kKeyFlagBits;
            ++col;
        }
        tcol[out + pos] = col - 1;
    }
    if (tid == 0) {
        first[total] = (uint32_t)T;
        tcount[(size_t)step * S + d] = total;
    }
    __syncthreads();
    const uint32_t pad_key = ((uint32_t)(e[0] >> 32) << kKeyFlagBits) | 1u;
    for (int j = tid; j < T; j += kMergeThreads) {
        const bool live = (uint32_t)j < total;
        tmult[out + j] = live ? (float)(first[j + 1] - first[j]) : 0.f;
        if (!live) tkey[out + j] = pad_key;
    }
}

void launch_merge_tails(const PlanShape& ps, const uint32_t* remote, const uint32_t* a2a, uint32_t* tkey,
                        float* tmult, uint32_t* tcol, uint32_t* tcount, hipStream_t stream) {
    hipLaunchKernelGGL(k_merge_tails, dim3(ps.S, ps.step_count), dim3(kMergeThreads), 0, stream, ps, remote, a2a,
                       tkey, tmult, tcol, tcount);
}

}  // namespace kge
