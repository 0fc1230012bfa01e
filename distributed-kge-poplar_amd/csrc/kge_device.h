// Device-side helpers shared by the kernel source files (element access, wave reductions,
// the tile order of the scoring launches, matrix-instruction vector types).
#pragma once

#include "kge_kernels.h"

#include <type_traits>

namespace kge {

#define DEVINL __device__ __forceinline__

// --------------------------------------------------------------------------
// element access

DEVINL float bf16_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
DEVINL uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// four consecutive elements starting at element k (k % 4 == 0) of a row
DEVINL float4 load4(const char* row, int k, int etype) {
    if (etype == ET_F32) return *reinterpret_cast<const float4*>(row + (size_t)k * 4);
    const uint2 raw = *reinterpret_cast<const uint2*>(row + (size_t)k * 2);
    if (etype == ET_BF16)
        return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u),
                           __uint_as_float(raw.y << 16), __uint_as_float(raw.y & 0xffff0000u));
    const __half2 h0 = *reinterpret_cast<const __half2*>(&raw.x);
    const __half2 h1 = *reinterpret_cast<const __half2*>(&raw.y);
    const float2 f0 = __half22float2(h0), f1 = __half22float2(h1);
    return make_float4(f0.x, f0.y, f1.x, f1.y);
}

DEVINL void store4(char* row, int k, int etype, float4 v) {
    if (etype == ET_F32) {
        *reinterpret_cast<float4*>(row + (size_t)k * 4) = v;
        return;
    }
    uint2 raw;
    if (etype == ET_BF16) {
        raw.x = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16);
        raw.y = (uint32_t)f32_to_bf16(v.z) | ((uint32_t)f32_to_bf16(v.w) << 16);
    } else {
        const __half2 h0 = __floats2half2_rn(v.x, v.y), h1 = __floats2half2_rn(v.z, v.w);
        raw.x = *reinterpret_cast<const uint32_t*>(&h0);
        raw.y = *reinterpret_cast<const uint32_t*>(&h1);
    }
    *reinterpret_cast<uint2*>(row + (size_t)k * 2) = raw;
}

// guarded variant for sources whose rows are not 16-byte aligned or whose
// length is not a multiple of four (standalone ops on arbitrary shapes)
DEVINL float4 round4_bf16(float4 v) {
    return make_float4(bf16_to_f32(f32_to_bf16(v.x)), bf16_to_f32(f32_to_bf16(v.y)),
                       bf16_to_f32(f32_to_bf16(v.z)), bf16_to_f32(f32_to_bf16(v.w)));
}
DEVINL float load1(const char* sec, int k, int etype) {
    if (etype == ET_F32) return reinterpret_cast<const float*>(sec)[k];
    if (etype == ET_BF16) return bf16_to_f32(reinterpret_cast<const uint16_t*>(sec)[k]);
    return __half2float(reinterpret_cast<const __half*>(sec)[k]);
}
DEVINL float4 load4(const char* row, int k, const RowSource& s) {
    if (s.vec) return load4(row, k, s.etype);
    float v[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) v[x] = (k + x < s.count) ? load1(row, k + x, s.etype) : 0.f;
    return make_float4(v[0], v[1], v[2], v[3]);
}

DEVINL const char* row_ptr(const RowSource& s, uint32_t r) {
    const uint32_t key = s.index ? s.index[r] : r;
    return s.base + (int64_t)key * s.pitch;
}

DEVINL float4 f4add(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
DEVINL float4 f4mul(float4 a, float4 b) { return make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w); }

// rel_mode: 0 none, 1 add (TransE), 2 multiply (DistMult)
DEVINL float4 combine_rel(float4 e, const float* relrow, int k, int rel_mode) {
    if (rel_mode == 0) return e;
    const float4 r = *reinterpret_cast<const float4*>(relrow + k);
    return rel_mode == 1 ? f4add(e, r) : f4mul(e, r);
}

DEVINL float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
// a wave-uniform float pinned to a scalar register
DEVINL float uniform_f32(float v) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v))); }
DEVINL float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}


// --------------------------------------------------------------------------
// Tile order.  The scoring kernels run gx * gy tiles for each of gz blocks; a
// block's tiles all read that block's operand rows (and coefficient matrix).
// Workgroups go to the 8 XCDs round-robin by linear id and every XCD has its own
// L2, so with the plain (x, y, z) order each XCD would fetch every block's
// operands.  Launching a 1-D grid and decoding it this way keeps a block's
// tiles on one XCD (block z on XCD z % 8), in consecutive slots of that XCD.
struct TileId { int x, y, z, gx, gy; };
constexpr int kXcdGroup = 2;
DEVINL TileId xcd_tile(int gx, int gy, int gz, int L) {
    const int n = gx * gy;
    int z, t;
    if ((gz & 7) == 0) {
        // kXcdGroup blocks of an XCD are interleaved tile by tile, so that the CUs of
        // an XCD do not all start on a new block's cold rows at the same moment
        const int j = L >> 3;
        const int G = ((gz >> 3) % kXcdGroup) == 0 ? kXcdGroup : 1;
        const int chunk = j / (G * n), r = j - chunk * (G * n);
        z = (L & 7) + 8 * (chunk * G + r % G);
        t = r / G;
    } else {
        z = L / n;
        t = L - z * n;
    }
    TileId id;
    id.y = t / gx; id.x = t - id.y * gx; id.z = z; id.gx = gx; id.gy = gy;
    return id;
}
DEVINL TileId xcd_tile(int gx, int gy, int gz) { return xcd_tile(gx, gy, gz, (int)blockIdx.x); }
static dim3 tile_grid(int gx, int gy, int gz) { return dim3((unsigned)(gx * gy * gz)); }


// f(integral_constant<0>) ... f(integral_constant<N-1>): a loop whose index is a compile-time constant
template <int N, int I = 0, class F>
DEVINL void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
DEVINL floatx4 as_x4(float4 v) { return floatx4{v.x, v.y, v.z, v.w}; }
DEVINL float4 as_f4(floatx4 v) { return make_float4(v.x, v.y, v.z, v.w); }

// float32 products from bfloat16 matrix instructions.  Every float32 value is
// the exact sum of three bfloat16 pieces (round to nearest of the value, of what
// that leaves, and of what that leaves: 8 + 8 + 8 significant bits), and
//   a * b = a0 b0 + (a0 b1 + a1 b0) + (a1 b1 + a0 b2 + a2 b0) + O(2^-24 |a b|):
// six v_mfma_f32_32x32x16_bf16 (float32 accumulate) per sixteen columns instead
// of eight v_mfma_f32_32x32x2_f32, at sixteen times the rate per instruction.
// Measured against float64 the sums are as accurate as the float32 instruction's.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
DEVINL uint32_t pack_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, bf16x2{(__bf16)a, (__bf16)b});
}
DEVINL float bf16_lo_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
DEVINL float bf16_hi_f32(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }
// four values -> their three pieces, four bfloat16 (8 bytes) per piece
DEVINL void split4_bf16(floatx4 v, uint2 piece[3]) {
    float r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int q = 0; q < 3; ++q) {
        const uint32_t p0 = pack_bf16(r[0], r[1]), p1 = pack_bf16(r[2], r[3]);
        piece[q] = make_uint2(p0, p1);
        if (q < 2) {
            r[0] -= bf16_lo_f32(p0); r[1] -= bf16_hi_f32(p0);
            r[2] -= bf16_lo_f32(p1); r[3] -= bf16_hi_f32(p1);
        }
    }
}
// the six products of one 16-column step, smallest first; a[q], b[q] hold piece q of
// eight consecutive columns of this lane's row
DEVINL floatx16 mfma_split6(const floatx4 a[3], const floatx4 b[3], floatx16 acc) {
#define KGE_MM(x_, y_)                                                                                \
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[x_]),                  \
                                                  __builtin_bit_cast(bf16x8, b[y_]), acc, 0, 0, 0)
    KGE_MM(0, 2); KGE_MM(2, 0); KGE_MM(1, 1); KGE_MM(0, 1); KGE_MM(1, 0); KGE_MM(0, 0);
#undef KGE_MM
    return acc;
}


constexpr int LDP = kScoreTile + 4;  // padded LDS row (floats), keeps float4 reads aligned
constexpr int BJ = 32;                // rows of `other` staged per iteration by the vector backward kernels

// scoring backward: out[i, k] = sum_j c[i, j] * phi(self[i, k], other[j, k]) (see kge_score_bwd.hip)
struct BwdParams {
    RowSource ent_a, ent_b;
    const float* rel;
    const uint32_t* crel;
    const float* coef;     // [S, B, T]
    const float* coef_div; // null, or [S, B, T]: coefficient = coef / coef_div, 0 where coef_div == 0
    float* grad;           // [R, Dp]
    int S, B, T, Dp;
    int side_b;            // 0: self = a-operand rows (heads), 1: self = b-operand rows (tails)
    int grad_c0;           // output row of block 0's first self row
    int vec_out;           // output rows allow aligned float4 stores
    int a_rel_mode;        // relation combine of the a-operand
    int a_c0, b_c0;
    int use_mfma;
    const uint32_t* nearflag;  // from the forward pass (L2 on the matrix cores), or null
    // merged tails (ScoreShape::tcount, tpad), or null: a block's b-operand rows end at tail_limit
    const uint32_t* tcount = nullptr;
    int tpad = 64;
    // optional rows added to the output (the feature projection's `embedding + ...`):
    // output row i gets row add_index[i] of add_base, row 0 for i >= *add_count
    const char* add_base;
    int64_t add_pitch;
    int add_etype;
    const uint32_t* add_index;
    const uint32_t* add_count;
};
void launch_bwd(const BwdParams& p, int dist_fn, hipStream_t stream);  // one side (p.side_b)

}  // namespace kge
