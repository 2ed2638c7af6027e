// Shared device/host helpers for the gfx950 Evoformer attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <float.h>
#include <stdint.h>

#include "evoattn.h"

#define EVO_CAT_(a, b) a##b
#define EVO_CAT(a, b) EVO_CAT_(a, b)

namespace evo {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
// A problem whose every key has a mask value below this is shifted by its largest mask
// value so that the log-sum-exp keeps its mantissa.
constexpr float kShiftThreshold = EVOATTN_SHIFT_THRESHOLD;
// Most negative additive mask value the matrix-core kernels carry (in log2 units).
constexpr float kMaskFloor = -1.0e30f;

// Launch-time constants derived on the host.
struct Extra {
    int n_chunks;      // number of S-chunks the dBias partials are split into
    int chunk;         // rows of S per chunk
    int vec_ok;        // bias rows may be read with 8/16-byte vector loads
    int bias_batches;  // 1 when one bias is shared by the whole batch, else B
    int bias_direct;   // the one-workgroup-per-problem kernels read the bias from the caller's tensor, not from bq / bk
    int dbias_chunks;  // > 0: the dK/dV kernel over a chunk of rows also sums that many dBias partials (else `dbias_reduce` does)
    int delta_given;   // `delta` already holds rowsum(dO * O) (the gate's pass wrote it): the dQ kernels read it and do not touch o
    // The gate's backward inside the dQ kernel over a chunk of rows (gate_dout non-null): that kernel stages the
    // gradient of the gated output, the gate's logits and the gated output, writes the gradient of the ungated
    // output to p.dout (for the dK/dV kernel) and the gate's gradient, and forms delta, as the gate's pass would.
    const void *gate_dout;   // gradient of the gated output, laid out like q
    const void *gate_logits;
    const void *gate_og;     // sigmoid(g) * O as the forward saved it
    void *gate_dgate;
    float *delta;      // [B][H][S][N]
    float *shift;      // [B][S] per-row mask shift (plain kernels)
    float *dbias_part; // [n_chunks][B][H][N][N]
    float *dmask_part; // [B][H][S][N]
    // prepared operands of the matrix-core kernels (written by the prep kernel)
    float *bq;         // bias * log2(e) in accumulator-tile order, lane = query  [Bb][H][NT][NT][64][16]
    float *bk;         // same, lane = key
    unsigned short *bq16;  // a bias in the dtype of q as given (16 bits, not scaled) in the same tile order, lane = query; else null
    unsigned short *bk16;  // same, lane = key
    uint2 *m2;         // additive mask * log2(e), shifted, clamped, as (hi, mid, lo, 0) of T  [B][S][NT*32]
    uint4 *m2a;        // the same mask rows as ready-made 16-byte operand chunks (hi, mid, lo, 1, 1, 1, 0, 0),
                       // padded with the floor to a multiple of 256 keys                        [B][S][NP256]
    void *bt;          // the bias transposed (key-major), in the dtype of q; null unless the bias has
                       // that dtype and N is a multiple of 8                                    [Bb][H][N][N]
    int *dead;         // [B][S] 1 where every key of the row is masked out
    int64_t zero_tile; // offset (elements) of an all-zero tile inside bq, bk, bq16 and bk16
    long long *trace;  // trace builds only: 16 timestamps per wave
};

// Rows of S per workgroup for a kernel that walks over a chunk of S rows of one of `base`
// (batch, head, query slab) items with one workgroup per CU at a time: n chunks run in
// ceil(base n / cus) rounds of ceil(S / n) rows.  A round also costs its start, its resident
// bias and the spread of its workgroups' finishing times, about three rows' worth, and a
// chunk `per_chunk` rows' worth (a partial result to write and sum again, where there is one).
// Returns the number of chunks with the smallest such count, among those of up to four rounds.
static inline int chunks_for_rounds(int64_t base, int S, int cus, double per_chunk) {
    if (base < 1) base = 1;
    const int64_t hi = (4 * (int64_t)cus + base - 1) / base;
    int64_t want = 1;
    double best = 1e30;
    for (int64_t n = 1; n <= hi && n <= S; ++n) {
        const int64_t rounds = (base * n + cus - 1) / cus, rows = (S + n - 1) / n;
        const double cost = (double)rounds * (double)rows + 3.0 * (double)rounds + per_chunk * (double)n;
        if (cost < best - 1e-9) { best = cost; want = n; }
    }
    return (int)want;
}

// Linear block id -> logical id such that consecutive logical ids run on one XCD
// (hardware deals consecutive workgroup ids round-robin over the 8 XCDs, each with its
// own L2).  Bijection on [0,total) for any total.
__device__ __forceinline__ unsigned xcd_remap(unsigned id, unsigned total) {
    constexpr unsigned X = 8;
    unsigned x = id % X, slot = id / X;
    unsigned q = total / X, r = total % X;
    return x * q + (x < r ? x : r) + slot;
}

struct Prob {
    int b, h, s;
    int64_t base;  // element offset of row 0 in the q-family tensors
    int64_t row0;  // offset of row 0 in lse / delta
};

__device__ __forceinline__ Prob decode_problem(const EvoAttnParams &p, unsigned pid) {
    Prob r;
    r.s = pid % p.S;
    unsigned t = pid / p.S;
    r.h = t % p.H;
    r.b = t / p.H;
    r.base = (int64_t)r.b * p.stride_b + (int64_t)r.h * p.stride_h + (int64_t)r.s * p.stride_s;
    r.row0 = (int64_t)pid * p.N;
    return r;
}

// The t-th problem in the order the one-workgroup-per-problem kernels walk them (consecutive t run on one XCD,
// behind one L2).  Where the heads lie inside a token (the per-head layout) and a head's row is shorter than a
// cache line, the line holds rows of several heads, and the heads of one (b, s) follow each other (bf16, forward /
// dK/dV in that layout: C5, 8 heads to a line, 335 -> 295 / 480 -> 405 us; C3, two to a line, 98 -> 94 / 127 ->
// 116 us; at C4's 768 keys 597 -> 608 / 770 -> 768 us, and head dim 64 loses 2 %: there and elsewhere a head's S
// rows follow each other).
__device__ __forceinline__ Prob walk_problem(const EvoAttnParams &p, unsigned t) {
    if (p.stride_h < p.stride_n && (p.D <= 16 || (p.D == 32 && p.N <= 512))) {
        const unsigned h = t % p.H, bs = t / p.H;
        return decode_problem(p, ((bs / p.S) * p.H + h) * p.S + bs % p.S);
    }
    return decode_problem(p, t);
}

// Additive form of mask[b][s][key]; -inf past the end of the row so that padded keys get
// zero probability whatever the rest of the row holds.
__device__ __forceinline__ float mask_add(const EvoAttnParams &p, int b, int s, int key) {
    if (key >= p.N) return -INFINITY;
    if (p.mask_kind == EVO_MASK_NONE) return 0.0f;
    int64_t off = (int64_t)b * p.mask_stride_b + (int64_t)s * p.mask_stride_s + key;
    switch (p.mask_kind) {
        case EVO_MASK_BOOL: return ((const uint8_t *)p.mask)[off] ? 0.0f : -FLT_MAX;
        case EVO_MASK_F32:  return ((const float *)p.mask)[off];
        case EVO_MASK_BF16: return (float)((const bf16_t *)p.mask)[off];
        default:            return (float)((const f16_t *)p.mask)[off];
    }
}

__device__ __forceinline__ float shift_from_max(float mx) { return mx < kShiftThreshold ? fmaxf(mx, -FLT_MAX) : 0.0f; }

// A bool keep-mask REPLACES the scores of dropped keys (evoformer.py:69, test.py:54), so no
// gradient reaches Q, K or the bias through them.  Where some key is kept the dropped keys
// have probability zero and that happens by itself; in a problem whose every key is dropped
// (shift != 0) the probabilities are uniform and dS has to be cleared explicitly.  dV, which
// does not pass through the scores, is unaffected.  Additive masks let the gradient through.
__device__ __forceinline__ bool ds_blocked(const EvoAttnParams &p, float shift) {
    return p.mask_kind == EVO_MASK_BOOL && shift != 0.0f;
}

// An int that every lane of the wave reads from the same address, written by an earlier
// kernel: through the constant address space, i.e. a scalar load.  As an ordinary load it
// would be a vector load, and waiting for it would also wait for every older vector store
// of the wave (vector memory operations complete in order).
__device__ __forceinline__ int uniform_load(const int *ptr) {
    return *(const __attribute__((address_space(4))) int *)(ptr);
}

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <typename T> struct Mfma;
template <> struct Mfma<bf16_t> {
    typedef bf16x8 v8;
    typedef bf16x4 v4;
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ f32x16 mma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mfma<f16_t> {
    typedef f16x8 v8;
    typedef f16x4 v4;
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ f32x16 mma(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// 32x32x16 MFMA operand / accumulator geometry used by every kernel (lane l, g = l / 32):
//   A (32 x 16): lane holds row l % 32, columns 8g .. 8g+7
//   B (16 x 32): lane holds column l % 32, rows 8g .. 8g+7
//   C (32 x 32): lane holds column l % 32, register r holds row 8*(r/4) + 4g + r%4
// A C tile is fed back as a B operand without any cross-lane traffic: k-step t takes
// registers 8t .. 8t+7, whose rows are crow(8t+i, g); the matching A operand must then list
// its columns in that row order, which acol_pos() gives as a storage position.
__device__ __forceinline__ int crow(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }
// position, inside a run of 32, at which row/key `x` is stored so that the 8 values one
// lane group needs for one k-step are contiguous: x = 16t + 8u + 4g + i -> 16t + 8g + 4u + i
__device__ __forceinline__ int perm_pos(int x) {
    return (x & ~15) | ((x & 4) << 1) | ((x & 8) >> 1) | (x & 3);
}

template <typename T>
__device__ __forceinline__ typename Mfma<T>::v8 ld8(const T *ptr) {
    return *reinterpret_cast<const typename Mfma<T>::v8 *>(ptr);
}
template <typename T>
__device__ __forceinline__ typename Mfma<T>::v8 zero8() {
    typename Mfma<T>::v8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (T)0.0f;
    return z;
}

// m = hi + mid + lo with all three representable in T: a fp32 value carried exactly (to
// 24 bits) through a 16-bit matrix-core operand.  fp16 cannot hold the mask floor; there
// the value is first clamped to what it can (a score that low has probability zero).
template <typename T>
__device__ __forceinline__ void split3(float m, T &hi, T &mid, T &lo) {
    hi = (T)m;
    const float r1 = m - (float)hi;
    mid = (T)r1;
    lo = (T)(r1 - (float)mid);
}
template <>
__device__ __forceinline__ void split3<f16_t>(float m, f16_t &hi, f16_t &mid, f16_t &lo) {
    m = fmaxf(m, -60000.0f);
    hi = (f16_t)m;
    const float r1 = m - (float)hi;
    mid = (f16_t)r1;
    lo = (f16_t)(r1 - (float)mid);
}

// raw * c as hi + lo, both representable in T: the product to 16 significant bits.
template <typename T>
__device__ __forceinline__ void scaled_hilo8(typename Mfma<T>::v8 raw, float c, typename Mfma<T>::v8 &hi,
                                             typename Mfma<T>::v8 &lo) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float f = (float)raw[i] * c;
        hi[i] = (T)f;
        lo[i] = (T)(f - (float)hi[i]);
    }
}

// acc + <a, b> over 8 elements of T, the products and sums in fp32 (`v_dot2c_f32_{bf16,f16}`:
// two elements per instruction and no conversions).
template <typename T>
__device__ __forceinline__ float dot8(typename Mfma<T>::v8 a, typename Mfma<T>::v8 b, float acc);
template <>
__device__ __forceinline__ float dot8<bf16_t>(bf16x8 a, bf16x8 b, float acc) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        bf2 x, y;
        x[0] = a[2 * i]; x[1] = a[2 * i + 1];
        y[0] = b[2 * i]; y[1] = b[2 * i + 1];
        acc = __builtin_amdgcn_fdot2_f32_bf16(x, y, acc, false);
    }
    return acc;
}
template <>
__device__ __forceinline__ float dot8<f16_t>(f16x8 a, f16x8 b, float acc) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        h2 x, y;
        x[0] = a[2 * i]; x[1] = a[2 * i + 1];
        y[0] = b[2 * i]; y[1] = b[2 * i + 1];
        acc = __builtin_amdgcn_fdot2(x, y, acc, false);
    }
    return acc;
}

// The two 16-bit values of a packed pair as fp32.
template <typename T>
__device__ __forceinline__ void unpack2(unsigned w, float &lo, float &hi);
template <>
__device__ __forceinline__ void unpack2<bf16_t>(unsigned w, float &lo, float &hi) {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
}
template <>
__device__ __forceinline__ void unpack2<f16_t>(unsigned w, float &lo, float &hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 v = __builtin_bit_cast(h2, w);
    lo = (float)v[0];
    hi = (float)v[1];
}

// A 32x32 bias tile as prepared in 16 bits: this lane's 16 accumulator entries, two to a
// register (entry 2 i in the low half of word i).  `unpack_tile16` gives them as fp32 times `mul`.
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
struct Tile16 {
    u32x4_t w[2];
};
__device__ __forceinline__ void load_tile16(const unsigned short *lane_tile, Tile16 &t) {
    t.w[0] = *reinterpret_cast<const u32x4_t *>(lane_tile);
    t.w[1] = *reinterpret_cast<const u32x4_t *>(lane_tile + 8);
}
template <typename T>
__device__ __forceinline__ void unpack_tile16(const Tile16 &t, float mul, f32x16 &dst) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float lo, hi;
        unpack2<T>(t.w[i >> 2][i & 3], lo, hi);
        dst[2 * i] = lo * mul;
        dst[2 * i + 1] = hi * mul;
    }
}

// A 32x32 bias tile in accumulator order, times `mul`, straight from the caller's tensor (for
// problems whose bias is used too few times to pay for the prepared fp32 tiles): `row` points
// at this lane's own bias row (lane = row of the matrix, the tile's 32 columns start at c0;
// entries 4 rr .. 4 rr + 3 are the columns c0 + 8 rr + 4 g ..).  The row must allow 16-byte
// (fp32) or 8-byte (16-bit) loads at multiples of four columns; groups past column n repeat
// the last whole group (such keys carry the mask floor).  F32: the tensor is fp32, else T.
template <typename T, bool F32>
__device__ __forceinline__ void bias_tile_rows(const void *row, int c0, int n, int g, float mul, f32x16 &dst) {
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const int col = min(c0 + 8 * rr + 4 * g, n - 4);
        if (F32) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>((const float *)row + col);
            dst[4 * rr] = v[0] * mul; dst[4 * rr + 1] = v[1] * mul; dst[4 * rr + 2] = v[2] * mul; dst[4 * rr + 3] = v[3] * mul;
        } else {
            const uint2 w = *reinterpret_cast<const uint2 *>((const T *)row + col);
            float f0, f1, f2, f3;
            unpack2<T>(w.x, f0, f1);
            unpack2<T>(w.y, f2, f3);
            dst[4 * rr] = f0 * mul; dst[4 * rr + 1] = f1 * mul; dst[4 * rr + 2] = f2 * mul; dst[4 * rr + 3] = f3 * mul;
        }
    }
}

// The same with lane = column of the matrix: `mat` points at element [0][0] (shared by the
// lanes), `col` is this lane's column, the tile's 32 rows start at r0, consecutive rows are
// `stride` elements apart (32-bit element offsets: the matrix has fewer than 2^31 entries); entry r
// is the row r0 + crow(r, g), rows past n - 1 repeat the last one.
template <typename T, bool F32>
__device__ __forceinline__ void bias_tile_cols(const void *mat, unsigned col, int r0, int n, unsigned stride, int g, float mul,
                                               f32x16 &dst) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const unsigned o = (unsigned)min(r0 + crow(r, g), n - 1) * stride + col;
        dst[r] = (F32 ? ((const float *)mat)[o] : (float)((const T *)mat)[o]) * mul;
    }
}

// (hi, mid, lo, 0) of split3 packed into 8 bytes.
template <typename T>
__device__ __forceinline__ uint2 pack_split3(float m) {
    T hi, mid, lo;
    split3<T>(m, hi, mid, lo);
    typename Mfma<T>::v4 v;
    v[0] = hi; v[1] = mid; v[2] = lo; v[3] = (T)0.0f;
    return __builtin_bit_cast(uint2, v);
}

// Four bias values for one query row and four consecutive keys, as fp32.
// BIASK: 0 none, 1 fp32, 2 same 16-bit type as T.
template <int BIASK, typename T>
__device__ __forceinline__ void load_bias4(const void *bias, int64_t off, int nvalid, bool vec, float out[4]) {
    if (BIASK == 0) {
        out[0] = out[1] = out[2] = out[3] = 0.0f;
    } else if (BIASK == 1) {
        const float *b = (const float *)bias + off;
        if (vec && nvalid >= 4) {
            f32x4 v = *reinterpret_cast<const f32x4 *>(b);
            out[0] = v[0]; out[1] = v[1]; out[2] = v[2]; out[3] = v[3];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = i < nvalid ? b[i] : 0.0f;
        }
    } else {
        const T *b = (const T *)bias + off;
        if (vec && nvalid >= 4) {
            typename Mfma<T>::v4 v = *reinterpret_cast<const typename Mfma<T>::v4 *>(b);
            out[0] = (float)v[0]; out[1] = (float)v[1]; out[2] = (float)v[2]; out[3] = (float)v[3];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = i < nvalid ? (float)b[i] : 0.0f;
        }
    }
}

template <int BIASK, typename T>
__device__ __forceinline__ float load_bias1(const void *bias, int64_t off) {
    if (BIASK == 0) return 0.0f;
    if (BIASK == 1) return ((const float *)bias)[off];
    return (float)((const T *)bias)[off];
}

// Store four consecutive fp32 values as T (8 bytes for 16-bit types).
template <typename T>
__device__ __forceinline__ void store4(T *dst, float a, float b, float c, float d) {
    typename Mfma<T>::v4 v;
    v[0] = (T)a; v[1] = (T)b; v[2] = (T)c; v[3] = (T)d;
    *reinterpret_cast<typename Mfma<T>::v4 *>(dst) = v;
}

// sigmoid(x) = 1 / (1 + 2^(-x log2 e)): one exp2 and one reciprocal.
__device__ __forceinline__ float sigmoidf(float x) { return __builtin_amdgcn_rcpf(1.0f + fast_exp2(-x * kLog2e)); }

// The output gate on one accumulator tile's worth of a row: acc[r] *= sigmoid(gate[column of r]).
// `grow` is this lane's row of the gate logits (laid out like the output row); a lane holds the
// columns c0 + 8 (r / 4) + 4 g + r % 4, four consecutive ones per load.
template <typename T>
__device__ __forceinline__ void gate_row_tile(const T *grow, int c0, int ncols, f32x16 &acc, int g) {
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const int c = c0 + 8 * rr + 4 * g;
        if (c < ncols) {
            const typename Mfma<T>::v4 v = *reinterpret_cast<const typename Mfma<T>::v4 *>(grow + c);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[4 * rr + i] *= sigmoidf((float)v[i]);
        }
    }
}

// One accumulator tile's worth of a row to memory as T: lane (li, g) holds, for its row, the
// 16 values of columns 8 (r / 4) + 4 g + r % 4; the two lanes of a row exchange halves so
// that each stores 16 contiguous bytes (columns c0 + 16 p + 8 g .. + 7, p = 0, 1) instead of
// four 8-byte pieces.  Columns at or beyond `ncols` are not stored.
template <typename T>
__device__ __forceinline__ void store_row_tile(T *row, int c0, int ncols, const f32x16 &acc, float scale, int g) {
#pragma unroll
    for (int pp = 0; pp < 2; ++pp) {
        typename Mfma<T>::v4 x, y;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[i] = (T)(acc[8 * pp + i] * scale);
            y[i] = (T)(acc[8 * pp + 4 + i] * scale);
        }
        const uint2 xu = __builtin_bit_cast(uint2, x), yu = __builtin_bit_cast(uint2, y);
        // lanes 32..63 of the first operand trade places with lanes 0..31 of the second
        auto s0 = __builtin_amdgcn_permlane32_swap(xu.x, yu.x, false, false);
        auto s1 = __builtin_amdgcn_permlane32_swap(xu.y, yu.y, false, false);
        const int c = c0 + 16 * pp + 8 * g;
        if (c < ncols) *reinterpret_cast<uint4 *>(row + c) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
    }
}

}  // namespace evo
