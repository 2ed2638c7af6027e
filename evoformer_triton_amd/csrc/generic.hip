// Plain kernels: every product and sum in fp32 on the vector ALU, one row per thread.
// They serve the fp32 "check mode" (EVO_F32), any head dim up to 128, any alignment, and
// are what the dispatcher falls back to when the matrix-core kernels do not cover a case.
//
// Arithmetic follows the reference kernels line by line in meaning, not in tiling:
// forward online softmax (evoformer.py:52-98, 285-297), delta (evoformer.py:313-323),
// dQ / dBias (evoformer.py:438-470), dK / dV (evoformer.py:575-619).
#include "common.h"
#include "kernels.h"

namespace evo {

template <typename T>
__device__ __forceinline__ void load_row(const T *src, float *dst, int D) {
    for (int d = 0; d < D; ++d) dst[d] = (float)src[d];
}

__device__ __forceinline__ float row_shift(const EvoAttnParams &p, int b, int s) {
    if (p.mask_kind == EVO_MASK_NONE) return 0.0f;
    float mx = -INFINITY;
    for (int j = 0; j < p.N; ++j) mx = fmaxf(mx, mask_add(p, b, s, j));
    return shift_from_max(mx);
}

// A row whose every key is masked below the shift threshold (shift != 0) takes its scores from the
// mask alone, as in the matrix-core kernels (prep.hip zeroes Q and the bias of such a row): the
// two families may serve the forward and the backward of one call, and the backward's
// exp(score - lse) is normalised only if both form the score the same way.  (Eager fp32
// arithmetic does the same by rounding once the mask is large enough to swamp q.k + bias.)
template <int BIASK, typename T>
__device__ __forceinline__ float score(const EvoAttnParams &p, float qk, int64_t bias_off, float mk, float shift) {
    if (shift != 0.0f) return mk - shift;
    return fmaf(qk, p.scale, load_bias1<BIASK, T>(p.bias, bias_off)) + mk;
}

template <typename T, int D, int BIASK>
__global__ void __launch_bounds__(64) gen_fwd(EvoAttnParams p) {
    const int nqb = (p.N + 63) / 64;
    const unsigned pid = blockIdx.x / nqb;
    const int row = (blockIdx.x % nqb) * 64 + threadIdx.x;
    const Prob pr = decode_problem(p, pid);
    const int rowc = row < p.N ? row : p.N - 1;
    const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
    float q[D], acc[D];
    load_row(Q + (int64_t)rowc * p.stride_n, q, D);
    for (int d = 0; d < D; ++d) acc[d] = 0.0f;
    const float shift = row_shift(p, pr.b, pr.s);
    const int64_t brow = (int64_t)pr.b * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h + (int64_t)rowc * p.bias_stride_row;
    float m = -INFINITY, l = 0.0f;
    for (int j = 0; j < p.N; ++j) {
        const T *kr = K + (int64_t)j * p.stride_n, *vr = V + (int64_t)j * p.stride_n;
        float qk = 0.0f;
        for (int d = 0; d < D; ++d) qk = fmaf(q[d], (float)kr[d], qk);
        float t = score<BIASK, T>(p, qk, brow + j, mask_add(p, pr.b, pr.s, j), shift);
        float mn = fmaxf(m, t);
        float alpha = expf(m - mn), pj = expf(t - mn);
        l = l * alpha + pj;
        for (int d = 0; d < D; ++d) acc[d] = fmaf(pj, (float)vr[d], acc[d] * alpha);
        m = mn;
    }
    if (row < p.N) {
        float inv = 1.0f / l;
        if (p.o) {   // (with a gate the caller may ask for the gated output alone)
            T *O = (T *)p.o + pr.base + (int64_t)row * p.stride_n;
            for (int d = 0; d < D; ++d) O[d] = (T)(acc[d] * inv);
        }
        if (p.gate) {
            const int64_t off = pr.base + (int64_t)row * p.stride_n;
            const T *Gt = (const T *)p.gate + off;
            T *Og = (T *)p.o_gated + off;
            for (int d = 0; d < D; ++d) Og[d] = (T)(acc[d] * inv / (1.0f + expf(-(float)Gt[d])));
        }
        p.lse[pr.row0 + row] = m + logf(l);
    }
}

template <typename T>
__global__ void __launch_bounds__(256) gen_delta(EvoAttnParams p, float *delta) {
    const int64_t rows = (int64_t)p.B * p.H * p.S * p.N;
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const Prob pr = decode_problem(p, (unsigned)(r / p.N));
    const int64_t off = pr.base + (r % p.N) * p.stride_n;
    const T *O = (const T *)p.o + off, *G = (const T *)p.dout + off;
    float s = 0.0f;
    for (int d = 0; d < p.D; ++d) s = fmaf((float)G[d], (float)O[d], s);
    delta[r] = s;
}

template <typename T, int D, int BIASK>
__global__ void __launch_bounds__(64) gen_dq(EvoAttnParams p, const float *delta, const float *shift_tab) {
    const int nqb = (p.N + 63) / 64;
    const unsigned pid = blockIdx.x / nqb;
    const int row = (blockIdx.x % nqb) * 64 + threadIdx.x;
    const Prob pr = decode_problem(p, pid);
    const int rowc = row < p.N ? row : p.N - 1;
    const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
    const T *G = (const T *)p.dout + pr.base;
    float q[D], g[D], acc[D];
    load_row(Q + (int64_t)rowc * p.stride_n, q, D);
    load_row(G + (int64_t)rowc * p.stride_n, g, D);
    for (int d = 0; d < D; ++d) acc[d] = 0.0f;
    const float shift = shift_tab[pr.b * p.S + pr.s];
    const bool kill = ds_blocked(p, shift);
    const float lse = p.lse[pr.row0 + rowc], dl = delta[pr.row0 + rowc];
    const int64_t brow = (int64_t)pr.b * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h + (int64_t)rowc * p.bias_stride_row;
    for (int j = 0; j < p.N; ++j) {
        const T *kr = K + (int64_t)j * p.stride_n, *vr = V + (int64_t)j * p.stride_n;
        float qk = 0.0f, dp = 0.0f;
        for (int d = 0; d < D; ++d) {
            qk = fmaf(q[d], (float)kr[d], qk);
            dp = fmaf(g[d], (float)vr[d], dp);
        }
        float t = score<BIASK, T>(p, qk, brow + j, mask_add(p, pr.b, pr.s, j), shift);
        float ds = kill ? 0.0f : expf(t - lse) * (dp - dl);
        for (int d = 0; d < D; ++d) acc[d] = fmaf(ds, (float)kr[d], acc[d]);
    }
    if (row < p.N) {
        T *dQ = (T *)p.dq + pr.base + (int64_t)row * p.stride_n;
        for (int d = 0; d < D; ++d) dQ[d] = (T)(acc[d] * p.scale);
    }
}

template <typename T, int D, int BIASK>
__global__ void __launch_bounds__(64) gen_dkdv(EvoAttnParams p, const float *delta, const float *shift_tab, float *dmask_part) {
    const int nkb = (p.N + 63) / 64;
    const unsigned pid = blockIdx.x / nkb;
    const int key = (blockIdx.x % nkb) * 64 + threadIdx.x;
    const Prob pr = decode_problem(p, pid);
    const int keyc = key < p.N ? key : p.N - 1;
    const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
    const T *G = (const T *)p.dout + pr.base;
    float k[D], v[D], dk[D], dv[D];
    load_row(K + (int64_t)keyc * p.stride_n, k, D);
    load_row(V + (int64_t)keyc * p.stride_n, v, D);
    for (int d = 0; d < D; ++d) dk[d] = dv[d] = 0.0f;
    const float shift = shift_tab[pr.b * p.S + pr.s];
    const bool kill = ds_blocked(p, shift);
    const float mk = mask_add(p, pr.b, pr.s, keyc);
    const int64_t bcol = (int64_t)pr.b * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h + keyc;
    float dm = 0.0f;
    for (int i = 0; i < p.N; ++i) {
        const T *qr = Q + (int64_t)i * p.stride_n, *gr = G + (int64_t)i * p.stride_n;
        float qk = 0.0f, dp = 0.0f;
        for (int d = 0; d < D; ++d) {
            qk = fmaf((float)qr[d], k[d], qk);
            dp = fmaf((float)gr[d], v[d], dp);
        }
        float t = score<BIASK, T>(p, qk, bcol + (int64_t)i * p.bias_stride_row, mk, shift);
        float pij = expf(t - p.lse[pr.row0 + i]);
        float ds = kill ? 0.0f : pij * (dp - delta[pr.row0 + i]);
        for (int d = 0; d < D; ++d) {
            dv[d] = fmaf(pij, (float)gr[d], dv[d]);
            dk[d] = fmaf(ds, (float)qr[d], dk[d]);
        }
        dm += ds;
    }
    if (key < p.N) {
        T *dK = (T *)p.dk + pr.base + (int64_t)key * p.stride_n;
        T *dV = (T *)p.dv + pr.base + (int64_t)key * p.stride_n;
        for (int d = 0; d < D; ++d) {
            dK[d] = (T)(dk[d] * p.scale);
            dV[d] = (T)dv[d];
        }
        if (dmask_part) dmask_part[pr.row0 + key] = dm;
    }
}

__device__ __forceinline__ void store_typed(void *dst, int dtype, int64_t i, float v) {
    if (dtype == EVO_F32) ((float *)dst)[i] = v;
    else if (dtype == EVO_BF16) ((bf16_t *)dst)[i] = (bf16_t)v;
    else ((f16_t *)dst)[i] = (f16_t)v;
}

// dBias[b,h,i,j] = sum over s of dS; one thread per element, s in order: deterministic.
template <typename T, int D, int BIASK>
__global__ void __launch_bounds__(64) gen_dbias(EvoAttnParams p, const float *delta, const float *shift_tab) {
    const int ncb = (p.N + 63) / 64;
    const int j = (blockIdx.x % ncb) * 64 + threadIdx.x;
    const unsigned t0 = blockIdx.x / ncb;
    const int i = t0 % p.N;
    const int h = (t0 / p.N) % p.H;
    const int b = t0 / p.N / p.H;
    if (j >= p.N) return;
    const int64_t boff = (int64_t)b * p.bias_stride_b + (int64_t)h * p.bias_stride_h + (int64_t)i * p.bias_stride_row + j;
    float acc = 0.0f;
    for (int s = 0; s < p.S; ++s) {
        const unsigned pid = ((unsigned)b * p.H + h) * p.S + s;
        const Prob pr = decode_problem(p, pid);
        const T *qr = (const T *)p.q + pr.base + (int64_t)i * p.stride_n;
        const T *gr = (const T *)p.dout + pr.base + (int64_t)i * p.stride_n;
        const T *kr = (const T *)p.k + pr.base + (int64_t)j * p.stride_n;
        const T *vr = (const T *)p.v + pr.base + (int64_t)j * p.stride_n;
        float qk = 0.0f, dp = 0.0f;
        for (int d = 0; d < D; ++d) {
            qk = fmaf((float)qr[d], (float)kr[d], qk);
            dp = fmaf((float)gr[d], (float)vr[d], dp);
        }
        const float shift = shift_tab[b * p.S + s];
        if (ds_blocked(p, shift)) continue;
        float t = score<BIASK, T>(p, qk, boff, mask_add(p, b, s, j), shift);
        acc += expf(t - p.lse[pr.row0 + i]) * (dp - delta[pr.row0 + i]);
    }
    store_typed(p.dbias, p.dbias_dtype, (((int64_t)b * p.H + h) * p.N + i) * p.N + j, acc);
}

// dMask[b,s,key] = sum over h of the per-problem column sums, h in order.
__global__ void __launch_bounds__(256) dmask_reduce(EvoAttnParams p, const float *part) {
    const int64_t n = (int64_t)p.B * p.S * p.N;
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const int key = t % p.N;
    const int s = (t / p.N) % p.S;
    const int b = t / p.N / p.S;
    float acc = 0.0f;
    for (int h = 0; h < p.H; ++h) acc += part[((((int64_t)b * p.H + h) * p.S) + s) * p.N + key];
    p.dmask[t] = acc;
}

// out[e] = sum over chunks of part[c][e], c in order; cast to the dBias dtype.
__global__ void __launch_bounds__(256) dbias_reduce(EvoAttnParams p, const float *part, int n_chunks) {
    const int64_t n = (int64_t)p.B * p.H * p.N * p.N;
    const int64_t t = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (t >= n) return;
    if ((n & 3) == 0) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int c = 0; c < n_chunks; ++c) acc += *reinterpret_cast<const f32x4 *>(part + (int64_t)c * n + t);
        for (int i = 0; i < 4; ++i) store_typed(p.dbias, p.dbias_dtype, t + i, acc[i]);
    } else {
        for (int64_t e = t; e < n && e < t + 4; ++e) {
            float acc = 0.0f;
            for (int c = 0; c < n_chunks; ++c) acc += part[(int64_t)c * n + e];
            store_typed(p.dbias, p.dbias_dtype, e, acc);
        }
    }
}

// shift[b][s] for the matrix-core backward kernels.
__global__ void __launch_bounds__(64) mask_shift_kernel(EvoAttnParams p, float *shift) {
    const int b = blockIdx.x / p.S, s = blockIdx.x % p.S;
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < p.N; j += 64) mx = fmaxf(mx, mask_add(p, b, s, j));
    mx = wave_max(mx);
    if (threadIdx.x == 0) shift[blockIdx.x] = p.mask_kind == EVO_MASK_NONE ? 0.0f : shift_from_max(mx);
}

// ---------------------------------------------------------------- host launchers

#define EVO_LAUNCH_CHECK()                                    \
    do {                                                      \
        hipError_t e_ = hipGetLastError();                    \
        if (e_ != hipSuccess) return EVO_EHIP - (int)e_;      \
    } while (0)

template <typename T, int D>
static int gen_fwd_bias(const EvoAttnParams &p, hipStream_t st) {
    const unsigned nqb = (p.N + 63) / 64, grid = nqb * (unsigned)(p.B * p.H * p.S);
    if (p.bias_dtype == EVO_NONE) gen_fwd<T, D, 0><<<grid, 64, 0, st>>>(p);
    else if (p.bias_dtype == EVO_F32) gen_fwd<T, D, 1><<<grid, 64, 0, st>>>(p);
    else gen_fwd<T, D, 2><<<grid, 64, 0, st>>>(p);
    EVO_LAUNCH_CHECK();
    return EVO_OK;
}

template <typename T, int D, int BIASK>
static int gen_bwd_launch(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const unsigned P = (unsigned)(p.B * p.H * p.S), nb = (p.N + 63) / 64;
    gen_dq<T, D, BIASK><<<nb * P, 64, 0, st>>>(p, e.delta, e.shift);
    EVO_LAUNCH_CHECK();
    gen_dkdv<T, D, BIASK><<<nb * P, 64, 0, st>>>(p, e.delta, e.shift, p.dmask ? e.dmask_part : nullptr);
    EVO_LAUNCH_CHECK();
    if (p.dbias) {
        gen_dbias<T, D, BIASK><<<nb * (unsigned)(p.B * p.H * p.N), 64, 0, st>>>(p, e.delta, e.shift);
        EVO_LAUNCH_CHECK();
    }
    return EVO_OK;
}

template <typename T, int D>
static int gen_bwd_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    if (p.bias_dtype == EVO_NONE) return gen_bwd_launch<T, D, 0>(p, e, st);
    if (p.bias_dtype == EVO_F32) return gen_bwd_launch<T, D, 1>(p, e, st);
    return gen_bwd_launch<T, D, 2>(p, e, st);
}

template <typename T>
static int gen_fwd_d(const EvoAttnParams &p, hipStream_t st) {
    switch (p.D) {
        case 8: return gen_fwd_bias<T, 8>(p, st);
        case 16: return gen_fwd_bias<T, 16>(p, st);
        case 32: return gen_fwd_bias<T, 32>(p, st);
        case 64: return gen_fwd_bias<T, 64>(p, st);
        case 128: return gen_fwd_bias<T, 128>(p, st);
    }
    return EVO_EUNSUPPORTED;
}

template <typename T>
static int gen_bwd_d(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    switch (p.D) {
        case 8: return gen_bwd_bias<T, 8>(p, e, st);
        case 16: return gen_bwd_bias<T, 16>(p, e, st);
        case 32: return gen_bwd_bias<T, 32>(p, e, st);
        case 64: return gen_bwd_bias<T, 64>(p, e, st);
        case 128: return gen_bwd_bias<T, 128>(p, e, st);
    }
    return EVO_EUNSUPPORTED;
}

int launch_generic_fwd(const EvoAttnParams &p, hipStream_t st) {
    switch (p.dtype) {
        case EVO_F32: return gen_fwd_d<float>(p, st);
        case EVO_BF16: return gen_fwd_d<bf16_t>(p, st);
        case EVO_F16: return gen_fwd_d<f16_t>(p, st);
    }
    return EVO_EINVAL;
}

int launch_delta_generic(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int64_t rows = (int64_t)p.B * p.H * p.S * p.N;
    const unsigned grid = (unsigned)((rows + 255) / 256);
    switch (p.dtype) {
        case EVO_F32: gen_delta<float><<<grid, 256, 0, st>>>(p, e.delta); break;
        case EVO_BF16: gen_delta<bf16_t><<<grid, 256, 0, st>>>(p, e.delta); break;
        default: gen_delta<f16_t><<<grid, 256, 0, st>>>(p, e.delta); break;
    }
    EVO_LAUNCH_CHECK();
    return EVO_OK;
}

// The gate's own backward, one pass over the rows: from the gradient of Og = sigmoid(g) * O (in
// p.dout), the gate logits g and the forward's output, gated (p.o_gated) or, where that is not
// given, ungated (p.o),
//     dO    = dout * sigmoid(g)                           -> dout_ungated (what the attention backward runs on)
//     dg    = dout * Og * (1 - sigmoid(g))                -> p.dgate       (= dout * O * sigmoid(g) * (1 - sigmoid(g)))
//     delta = sum over the head dim of dO * (Og / sigmoid(g)) -> delta      (= rowsum(dO * O), with dO as stored)
// the first two laid out like q, delta [B][H][S][N].  With delta formed here the dQ kernels need no
// ungated O, so the forward need not write one.  One thread per 8 consecutive head-dim elements of
// one row at a time; the D / 8 threads of a row are neighbours in a wave and add their parts of delta.
//
// A workgroup takes 32 tokens of one S row with all their heads, in the order the pieces lie in memory
// (heads inside a token: (token, head, piece); else (head, token, piece)), and writes its 32 x H sums of
// delta from LDS, 128 bytes per head (from the threads that form them they would go out as single floats
// S * N * 4 bytes apart).  The pass moves five tensors of q's size, three in and two out, and runs at the
// speed of the memory: S = 512, N = 256, H = 8, head dim 32 in bf16 is 340 MB in 65..68 us, 5 TB/s.
template <typename T, bool FROM_GATED>
__global__ void __launch_bounds__(256) gate_bwd_kernel(EvoAttnParams p, T *dout_ungated, float *delta, int sh_c) {
    extern __shared__ float gate_sums[];   // [H][32]
    const unsigned cpr = 1u << sh_c;       // 8-element pieces per row of D (1, 2, 4, 8 or 16)
    // blockIdx.y, .z: the S row of the batch (z * gridDim.y + y = b * S + s)
    const unsigned bs = blockIdx.z * gridDim.y + blockIdx.y;
    if (bs >= (unsigned)p.B * (unsigned)p.S) return;   // uniform over the workgroup
    const int b = (int)(bs / (unsigned)p.S), s = (int)(bs - (unsigned)b * (unsigned)p.S);
    const unsigned n0 = blockIdx.x * 32u, ntok = min(32u, (unsigned)p.N - n0), H = (unsigned)p.H;
    const bool tokens = p.stride_h < p.stride_n;
    const unsigned inner = tokens ? H : ntok;
    const unsigned total = ntok * H * cpr;
    const int64_t base = (int64_t)b * p.stride_b + (int64_t)s * p.stride_s + (int64_t)n0 * p.stride_n;
    // eight elements at a time: 16-byte loads and stores for the 16-bit types (the pieces are
    // 16-byte aligned: dense tensors, head dim a multiple of 8), two of each for fp32
    constexpr int V = sizeof(T) == 2 ? 8 : 4;
    typedef T vec __attribute__((ext_vector_type(V)));
    for (unsigned i00 = 0; i00 < total; i00 += 256) {   // uniform
        const unsigned i0 = i00 + threadIdx.x;
        const unsigned i = i0 < total ? i0 : total - 1;   // (the threads past the end keep the row sums below whole)
        const unsigned c = i & (cpr - 1), r = i >> sh_c;
        const unsigned outer_i = r / inner, inner_i = r - outer_i * inner;
        const unsigned h = tokens ? inner_i : outer_i, tk = tokens ? outer_i : inner_i;
        const int64_t off = base + (int64_t)tk * p.stride_n + (int64_t)h * p.stride_h + c * 8;
        const T *go = (const T *)p.dout + off, *gl = (const T *)p.gate + off;
        const T *o = (const T *)(FROM_GATED ? p.o_gated : p.o) + off;
        T *d_o = dout_ungated + off, *d_g = (T *)p.dgate + off;
        float dsum = 0.0f;
#pragma unroll
        for (int j0 = 0; j0 < 8; j0 += V) {
            const vec a = *reinterpret_cast<const vec *>(go + j0), b2 = *reinterpret_cast<const vec *>(gl + j0),
                      c2 = *reinterpret_cast<const vec *>(o + j0);
            vec r_o, r_g;
#pragma unroll
            for (int j = 0; j < V; ++j) {
                // (the 16-bit types take the hardware's exp2 and reciprocal, one ulp each, as the MFMA forward does)
                const float den = 1.0f + (sizeof(T) == 4 ? expf(-(float)b2[j]) : fast_exp2(-(float)b2[j] * kLog2e));
                const float sg = sizeof(T) == 4 ? 1.0f / den : __builtin_amdgcn_rcpf(den);
                const float gr = (float)a[j];
                const float og = FROM_GATED ? (float)c2[j] : (float)c2[j] * sg;   // sigmoid(g) * O
                r_o[j] = (T)(gr * sg);
                r_g[j] = (T)(gr * og * (1.0f - sg));
                // delta from the dO that the attention backward will read, rounded as it is stored, against
                // O = Og / sigmoid(g): dP is formed from the same rounded dO, and in dS = P (dP - delta) the
                // rounding of dO then cancels as far as P is peaked (with delta from dout * Og it does not)
                dsum = fmaf((float)r_o[j], FROM_GATED ? (float)c2[j] * den : (float)c2[j], dsum);
            }
            if (i0 < total) {
                *reinterpret_cast<vec *>(d_o + j0) = r_o;
                *reinterpret_cast<vec *>(d_g + j0) = r_g;
            }
        }
        for (unsigned w = 1; w < cpr; w <<= 1) dsum += __shfl_xor(dsum, (int)w);
        if (c == 0 && i0 < total) gate_sums[h * 32 + tk] = dsum;
    }
    __syncthreads();
    for (unsigned j = threadIdx.x; j < H * 32; j += 256) {
        const unsigned h = j >> 5, tk = j & 31;
        if (tk < ntok) delta[(((int64_t)b * p.H + h) * p.S + s) * p.N + n0 + tk] = gate_sums[j];
    }
}

int launch_gate_bwd(const EvoAttnParams &p, void *dout_ungated, float *delta, hipStream_t st) {
    const int cpr = p.D / 8;
    int sh_c = 0;
    while ((1 << sh_c) < cpr) ++sh_c;
    const int64_t rows = (int64_t)p.B * p.S;
    // (head dims are 8 .. 128 in powers of two; 128 bytes of LDS per head)
    if ((1 << sh_c) != cpr || rows > (int64_t)32768 * 65535 || p.H > 256) return EVO_EUNSUPPORTED;
    const unsigned gy = (unsigned)(rows < 32768 ? rows : 32768);
    const dim3 grid((unsigned)((p.N + 31) / 32), gy, (unsigned)((rows + gy - 1) / gy));
    const size_t lds = (size_t)p.H * 32 * sizeof(float);
    const bool g = p.o_gated != nullptr;
    if (p.dtype == EVO_F32) {
        if (g) gate_bwd_kernel<float, true><<<grid, 256, lds, st>>>(p, (float *)dout_ungated, delta, sh_c);
        else gate_bwd_kernel<float, false><<<grid, 256, lds, st>>>(p, (float *)dout_ungated, delta, sh_c);
    } else if (p.dtype == EVO_BF16) {
        if (g) gate_bwd_kernel<bf16_t, true><<<grid, 256, lds, st>>>(p, (bf16_t *)dout_ungated, delta, sh_c);
        else gate_bwd_kernel<bf16_t, false><<<grid, 256, lds, st>>>(p, (bf16_t *)dout_ungated, delta, sh_c);
    } else {
        if (g) gate_bwd_kernel<f16_t, true><<<grid, 256, lds, st>>>(p, (f16_t *)dout_ungated, delta, sh_c);
        else gate_bwd_kernel<f16_t, false><<<grid, 256, lds, st>>>(p, (f16_t *)dout_ungated, delta, sh_c);
    }
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

int launch_dmask_reduce(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int64_t n = (int64_t)p.B * p.S * p.N;
    dmask_reduce<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(p, e.dmask_part);
    EVO_LAUNCH_CHECK();
    return EVO_OK;
}

int launch_dbias_reduce(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int64_t n = ((int64_t)p.B * p.H * p.N * p.N + 3) / 4;
    dbias_reduce<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(p, e.dbias_part, e.n_chunks);
    EVO_LAUNCH_CHECK();
    return EVO_OK;
}

int launch_mask_shift(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    mask_shift_kernel<<<(unsigned)(p.B * p.S), 64, 0, st>>>(p, e.shift);
    EVO_LAUNCH_CHECK();
    return EVO_OK;
}

int launch_generic_bwd(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    int rc = e.delta_given ? EVO_OK : launch_delta_generic(p, e, st);
    if (rc) return rc;
    rc = launch_mask_shift(p, e, st);
    if (rc) return rc;
    switch (p.dtype) {
        case EVO_F32: rc = gen_bwd_d<float>(p, e, st); break;
        case EVO_BF16: rc = gen_bwd_d<bf16_t>(p, e, st); break;
        case EVO_F16: rc = gen_bwd_d<f16_t>(p, e, st); break;
        default: rc = EVO_EINVAL;
    }
    if (rc) return rc;
    if (p.dmask) rc = launch_dmask_reduce(p, e, st);
    return rc;
}

}  // namespace evo
