// Backward kernels for gfx950 on the bf16/fp16 32x32x16 matrix-core instruction.
// Compiled once per head dim (-DEVO_D=8|16|32|64).
//
// They replace the reference's `_attn_bwd_preprocess` (evoformer.py:299-326),
// `_attn_bwd_dq` (:329-476) and `_attn_bwd_dk_dv` (:479-630).  Both big kernels recompute
// P = exp(score - LSE) from the saved log-sum-exp (:452, :600), form
// dS = P * (dP - delta) (:456, :610) and cast P and dS to the input dtype before the
// gradient matmuls (:459, :603, :611); dQ and dK are multiplied by the softmax scale after
// the matmul (:462, :614).
//
// dBias is the sum of dS over S.  The reference adds every fp32 dS tile into global memory
// with atomics (:458).  Here the dQ kernel owns a 32-query slab of one head for a whole
// chunk of S rows and keeps the running sum of dS for that slab in matrix-core
// accumulators (an identity-matrix MFMA adds the bf16 dS tile that the dQ matmul consumes
// anyway), writes one partial per chunk, and a second kernel adds the partials in a fixed
// order: no floating-point atomics, bit-reproducible.
#include "common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

// delta[row] = sum_d dO[row,d] * O[row,d]  (evoformer.py:313-323)
template <typename T, int D>
__global__ void __launch_bounds__(256) mfma_delta(EvoAttnParams p, float *delta) {
    typedef typename Mfma<T>::v8 v8;
    const int64_t rows = (int64_t)p.B * p.H * p.S * p.N;
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    const Prob pr = decode_problem(p, (unsigned)(r / p.N));
    const int64_t off = pr.base + (r % p.N) * p.stride_n;
    const T *O = (const T *)p.o + off, *G = (const T *)p.dout + off;
    float s = 0.0f;
#pragma unroll
    for (int c = 0; c < D / 8; ++c) {
        v8 o = ld8(O + c * 8), g = ld8(G + c * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) s = fmaf((float)g[i], (float)o[i], s);
    }
    delta[r] = s;
}

// ------------------------------------------------------------------ dQ and dBias partials
//
// Workgroup = 4 waves = (b, h, chunk of S, 32 query rows).  The waves split the keys:
// wave w takes 32-key tiles w, w+4, w+8, ...  Scores are computed transposed
// (S^T = K Q^T, dP^T = V dO^T) so that a lane owns one query and 16 keys, which makes the
// dS^T accumulator tile the B operand of both dQ^T += K^T dS^T and dBias^T += I dS^T.
// Each wave's partial dQ^T meets the others in LDS once per S row and is summed in wave
// order.
template <typename T, int D, int BIASK, int NTW>
__global__ void __launch_bounds__(256) mfma_dq(EvoAttnParams p, Extra e) {
    constexpr int DK = D < 16 ? 16 : D;
    constexpr int KS = DK / 16;
    constexpr int DT = (D + 31) / 32;
    constexpr int RP = DT * 32 + 4;  // pitch of a partial dQ row in LDS (floats)
    typedef typename Mfma<T>::v8 v8;

    __shared__ __attribute__((aligned(16))) float Ms[NTW * 128];
    __shared__ __attribute__((aligned(16))) float red[4 * 32 * RP];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const int qt = lid % NT;
    const unsigned bh = (lid / NT) % (unsigned)(p.B * p.H);
    const int c = lid / NT / (unsigned)(p.B * p.H);
    const int b = bh / p.H, h = bh % p.H;
    const int q0 = qt * 32;
    const int qrow = min(q0 + li, p.N - 1);
    const int64_t sn = p.stride_n;
    const int64_t brow = (int64_t)b * p.bias_stride_b + (int64_t)h * p.bias_stride_h + (int64_t)qrow * p.bias_stride_row;
    const bool vec = e.vec_ok != 0;
    const bool want_dbias = e.dbias_part != nullptr && p.dbias != nullptr;
    const float scale = p.scale;

    // identity slices: A[m][8g+i] = 1 where m is the key row that register 8ts+i of a
    // C-layout tile holds for lane group g
    v8 idf[2];
#pragma unroll
    for (int ts = 0; ts < 2; ++ts)
#pragma unroll
        for (int i = 0; i < 8; ++i) idf[ts][i] = (T)(li == crow(8 * ts + i, g) ? 1.0f : 0.0f);

    f32x16 dbacc[NTW];
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) dbacc[j][r] = 0.0f;

    const int s_begin = c * e.chunk, s_end = min(p.S, s_begin + e.chunk);
    for (int s = s_begin; s < s_end; ++s) {
        const unsigned pid = (bh * (unsigned)p.S) + s;
        const Prob pr = decode_problem(p, pid);
        const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
        const T *G = (const T *)p.dout + pr.base;

        __syncthreads();  // last row's readers of Ms and red are done
        for (int j = tid; j < NTW * 128; j += 256) Ms[j] = mask_add(p, b, s, j);
        const float shift = e.shift[b * p.S + s];
        v8 qf[KS], gf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 16 + g * 8;
            qf[ks] = d0 < D ? ld8(Q + (int64_t)qrow * sn + d0) : zero8<T>();
            gf[ks] = d0 < D ? ld8(G + (int64_t)qrow * sn + d0) : zero8<T>();
        }
        const float lse = p.lse[pr.row0 + qrow], dl = e.delta[pr.row0 + qrow];
        __syncthreads();

        f32x16 dqacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dqacc[dt][r] = 0.0f;

#pragma unroll 1
        for (int j = 0; j < NTW; ++j) {
            const int kt = wave + 4 * j;
            if (kt * 32 < p.N) {  // wave-uniform
                const int kb = kt * 32;
                const int keyc = min(kb + li, p.N - 1);
                f32x16 acc, dp;
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = dp[r] = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int d0 = ks * 16 + g * 8;
                    v8 ka = d0 < D ? ld8(K + (int64_t)keyc * sn + d0) : zero8<T>();
                    v8 va = d0 < D ? ld8(V + (int64_t)keyc * sn + d0) : zero8<T>();
                    acc = Mfma<T>::mma(ka, qf[ks], acc);
                    dp = Mfma<T>::mma(va, gf[ks], dp);
                }
                float ds[16];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int kg = kb + 8 * rr + 4 * g;
                    float bv[4];
                    load_bias4<BIASK, T>(p.bias, brow + kg, p.N - kg, vec, bv);
                    const f32x4 mk = *reinterpret_cast<const f32x4 *>(&Ms[kg]);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float t = fmaf(acc[4 * rr + i], scale, bv[i]) + mk[i];
                        if (shift != 0.0f) t -= shift;
                        const float pv = fast_exp2((t - lse) * kLog2e);
                        ds[4 * rr + i] = pv * (dp[4 * rr + i] - dl);
                    }
                }
#pragma unroll
                for (int ts = 0; ts < 2; ++ts) {
                    v8 dsf;
#pragma unroll
                    for (int i = 0; i < 8; ++i) dsf[i] = (T)ds[8 * ts + i];
                    if (want_dbias) {
                        // j is a run-time value here; the compare chain keeps the
                        // accumulator index static so the tiles stay in registers
#pragma unroll
                        for (int jj = 0; jj < NTW; ++jj)
                            if (jj == j) dbacc[jj] = Mfma<T>::mma(idf[ts], dsf, dbacc[jj]);
                    }
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        // K^T operand: row d, columns = the keys registers 8ts..8ts+7 hold
                        const int d = dt * 32 + li;
                        v8 kta;
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            const int key = min(kb + crow(8 * ts + i, g), p.N - 1);
                            kta[i] = d < D ? K[(int64_t)key * sn + d] : (T)0.0f;
                        }
                        dqacc[dt] = Mfma<T>::mma(kta, dsf, dqacc[dt]);
                    }
                }
            }
        }

        // partial dQ^T of this wave: lane = query li, register r = dim dt*32 + crow(r, g)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                f32x4 v;
                v[0] = dqacc[dt][4 * rr]; v[1] = dqacc[dt][4 * rr + 1];
                v[2] = dqacc[dt][4 * rr + 2]; v[3] = dqacc[dt][4 * rr + 3];
                *reinterpret_cast<f32x4 *>(&red[(wave * 32 + li) * RP + dt * 32 + 8 * rr + 4 * g]) = v;
            }
        __syncthreads();
        T *dQ = (T *)p.dq + pr.base;
        for (int it = tid; it < 32 * (D / 4); it += 256) {
            const int q = it / (D / 4), d4 = (it % (D / 4)) * 4;
            f32x4 sum = *reinterpret_cast<const f32x4 *>(&red[q * RP + d4]);
#pragma unroll
            for (int w = 1; w < 4; ++w) sum += *reinterpret_cast<const f32x4 *>(&red[(w * 32 + q) * RP + d4]);
            if (q0 + q < p.N)
                store4<T>(dQ + (int64_t)(q0 + q) * sn + d4, sum[0] * scale, sum[1] * scale, sum[2] * scale, sum[3] * scale);
        }
    }

    if (want_dbias && q0 + li < p.N) {
        float *part = e.dbias_part + ((((int64_t)c * p.B + b) * p.H + h) * p.N + (q0 + li)) * p.N;
        const bool v4ok = (p.N & 3) == 0;
#pragma unroll
        for (int j = 0; j < NTW; ++j) {
            const int kb = (wave + 4 * j) * 32;
            if (kb < p.N) {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int kg = kb + 8 * rr + 4 * g;
                    if (v4ok && kg + 4 <= p.N) {
                        f32x4 v;
                        v[0] = dbacc[j][4 * rr]; v[1] = dbacc[j][4 * rr + 1];
                        v[2] = dbacc[j][4 * rr + 2]; v[3] = dbacc[j][4 * rr + 3];
                        *reinterpret_cast<f32x4 *>(part + kg) = v;
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                            if (kg + i < p.N) part[kg + i] = dbacc[j][4 * rr + i];
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------ dK, dV (and dMask partials)
//
// Workgroup = 4 waves = 128 keys of one problem; each wave keeps its 32 keys' K and V
// operands in registers and loops over all query rows, staged 64 at a time through LDS both
// row-major (for S = Q K^T, dP = dO V^T) and transposed (for dV^T += dO^T P, dK^T += Q^T dS).
// Scores are NOT transposed here: a lane owns one key and 16 queries, so that P and dS in
// accumulator layout are the B operands of the two gradient matmuls.
template <typename T, int D, int BIASK>
__global__ void __launch_bounds__(256) mfma_dkdv(EvoAttnParams p, Extra e) {
    constexpr int BK = 128, BQS = 64;
    constexpr int DK = D < 16 ? 16 : D;
    constexpr int KS = DK / 16;
    constexpr int DT = (D + 31) / 32;
    constexpr int DP = DT * 32;
    constexpr int QP = DK + 8;
    constexpr int TP = BQS + 8;
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v2 v2;

    __shared__ __attribute__((aligned(16))) T Qs[BQS * QP];
    __shared__ __attribute__((aligned(16))) T Gs[BQS * QP];
    __shared__ __attribute__((aligned(16))) T Qt[DP * TP];
    __shared__ __attribute__((aligned(16))) T Gt[DP * TP];
    __shared__ __attribute__((aligned(16))) float Ls[BQS];
    __shared__ __attribute__((aligned(16))) float Ds[BQS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, g = lane >> 5;
    const int nkb = (p.N + BK - 1) / BK;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const unsigned pid = lid / nkb;
    const int key0 = (lid % nkb) * BK + wave * 32;
    const Prob pr = decode_problem(p, pid);
    const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
    const T *G = (const T *)p.dout + pr.base;
    const int64_t sn = p.stride_n;
    const bool active = key0 < p.N;
    const int key = key0 + li, keyc = min(key, p.N - 1);
    const float scale = p.scale;

    for (int i = tid; i < BQS * QP; i += 256) Qs[i] = Gs[i] = (T)0.0f;
    for (int i = tid; i < DP * TP; i += 256) Qt[i] = Gt[i] = (T)0.0f;

    v8 kf[KS], vf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = ks * 16 + g * 8;
        kf[ks] = d0 < D ? ld8(K + (int64_t)keyc * sn + d0) : zero8<T>();
        vf[ks] = d0 < D ? ld8(V + (int64_t)keyc * sn + d0) : zero8<T>();
    }
    const float mk = mask_add(p, pr.b, pr.s, key);
    const float shift = e.shift[pr.b * p.S + pr.s];
    const int64_t bcol = (int64_t)pr.b * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h + keyc;
    const bool want_dm = e.dmask_part != nullptr && p.dmask != nullptr;

    f32x16 dk[DT], dv[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dk[dt][r] = dv[dt][r] = 0.0f;
    float dm = 0.0f;

    for (int qs0 = 0; qs0 < p.N; qs0 += BQS) {
        __syncthreads();
        for (int it = tid; it < BQS * (D / 8); it += 256) {
            const int row = it / (D / 8), c = it % (D / 8), qq = qs0 + row;
            v8 a = qq < p.N ? ld8(Q + (int64_t)qq * sn + c * 8) : zero8<T>();
            v8 bb = qq < p.N ? ld8(G + (int64_t)qq * sn + c * 8) : zero8<T>();
            *reinterpret_cast<v8 *>(&Qs[row * QP + c * 8]) = a;
            *reinterpret_cast<v8 *>(&Gs[row * QP + c * 8]) = bb;
        }
        for (int it = tid; it < (BQS / 2) * (D / 8); it += 256) {
            const int jp = it / (D / 8), c = it % (D / 8), r0 = qs0 + 2 * jp;
            v8 qa = r0 < p.N ? ld8(Q + (int64_t)r0 * sn + c * 8) : zero8<T>();
            v8 qb = r0 + 1 < p.N ? ld8(Q + (int64_t)(r0 + 1) * sn + c * 8) : zero8<T>();
            v8 ga = r0 < p.N ? ld8(G + (int64_t)r0 * sn + c * 8) : zero8<T>();
            v8 gb = r0 + 1 < p.N ? ld8(G + (int64_t)(r0 + 1) * sn + c * 8) : zero8<T>();
            const int pos = perm_pos(2 * jp);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v2 w;
                w[0] = qa[i]; w[1] = qb[i];
                *reinterpret_cast<v2 *>(&Qt[(c * 8 + i) * TP + pos]) = w;
                w[0] = ga[i]; w[1] = gb[i];
                *reinterpret_cast<v2 *>(&Gt[(c * 8 + i) * TP + pos]) = w;
            }
        }
        if (tid < BQS) {
            const int qq = qs0 + tid;
            Ls[tid] = qq < p.N ? p.lse[pr.row0 + qq] : INFINITY;
            Ds[tid] = qq < p.N ? e.delta[pr.row0 + qq] : 0.0f;
        }
        __syncthreads();

        if (active) {
#pragma unroll
            for (int qt = 0; qt < BQS / 32; ++qt) {
                const int qb = qt * 32;
                if (qs0 + qb >= p.N) break;
                f32x16 acc, dp;
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = dp[r] = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    v8 qa = *reinterpret_cast<const v8 *>(&Qs[(qb + li) * QP + ks * 16 + g * 8]);
                    v8 ga = *reinterpret_cast<const v8 *>(&Gs[(qb + li) * QP + ks * 16 + g * 8]);
                    acc = Mfma<T>::mma(qa, kf[ks], acc);
                    dp = Mfma<T>::mma(ga, vf[ks], dp);
                }
                float pv[16], ds[16];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int ql = qb + 8 * rr + 4 * g;
                    const f32x4 l4 = *reinterpret_cast<const f32x4 *>(&Ls[ql]);
                    const f32x4 d4 = *reinterpret_cast<const f32x4 *>(&Ds[ql]);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int qg = min(qs0 + ql + i, p.N - 1);
                        const float bv = load_bias1<BIASK, T>(p.bias, bcol + (int64_t)qg * p.bias_stride_row);
                        float t = fmaf(acc[4 * rr + i], scale, bv) + mk;
                        if (shift != 0.0f) t -= shift;
                        pv[4 * rr + i] = fast_exp2((t - l4[i]) * kLog2e);
                        ds[4 * rr + i] = pv[4 * rr + i] * (dp[4 * rr + i] - d4[i]);
                    }
                }
                if (want_dm) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) dm += ds[r];
                }
#pragma unroll
                for (int ts = 0; ts < 2; ++ts) {
                    v8 pf, dsf;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        pf[i] = (T)pv[8 * ts + i];
                        dsf[i] = (T)ds[8 * ts + i];
                    }
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        v8 ga = *reinterpret_cast<const v8 *>(&Gt[(dt * 32 + li) * TP + qb + ts * 16 + g * 8]);
                        v8 qa = *reinterpret_cast<const v8 *>(&Qt[(dt * 32 + li) * TP + qb + ts * 16 + g * 8]);
                        dv[dt] = Mfma<T>::mma(ga, pf, dv[dt]);
                        dk[dt] = Mfma<T>::mma(qa, dsf, dk[dt]);
                    }
                }
            }
        }
    }

    if (active) {
        if (want_dm) {
            dm += __shfl_xor(dm, 32);
            if (g == 0 && key < p.N) e.dmask_part[pr.row0 + key] = dm;
        }
        if (key < p.N) {
            T *dK = (T *)p.dk + pr.base + (int64_t)key * sn;
            T *dV = (T *)p.dv + pr.base + (int64_t)key * sn;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int d0 = dt * 32 + 8 * rr + 4 * g;
                    if (d0 < D) {
                        store4<T>(dK + d0, dk[dt][4 * rr] * scale, dk[dt][4 * rr + 1] * scale,
                                  dk[dt][4 * rr + 2] * scale, dk[dt][4 * rr + 3] * scale);
                        store4<T>(dV + d0, dv[dt][4 * rr], dv[dt][4 * rr + 1], dv[dt][4 * rr + 2], dv[dt][4 * rr + 3]);
                    }
                }
        }
    }
}

// ------------------------------------------------------------------ launchers

static inline int hip_rc() {
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

template <typename T, int D, int BIASK>
static int dq_ntw(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int NT = (p.N + 31) / 32;
    const unsigned grid = (unsigned)NT * (unsigned)(p.B * p.H) * (unsigned)e.n_chunks;
    const int ntw = (NT + 3) / 4;
    if (ntw <= 2) mfma_dq<T, D, BIASK, 2><<<grid, 256, 0, st>>>(p, e);
    else if (ntw <= 4) mfma_dq<T, D, BIASK, 4><<<grid, 256, 0, st>>>(p, e);
    else if (ntw <= 8) mfma_dq<T, D, BIASK, 8><<<grid, 256, 0, st>>>(p, e);
    else if (ntw <= 16) mfma_dq<T, D, BIASK, 16><<<grid, 256, 0, st>>>(p, e);
    else return EVO_EUNSUPPORTED;
    return hip_rc();
}

template <typename T, int D>
static int dq_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    if (p.bias_dtype == EVO_NONE) return dq_ntw<T, D, 0>(p, e, st);
    if (p.bias_dtype == EVO_F32) return dq_ntw<T, D, 1>(p, e, st);
    return dq_ntw<T, D, 2>(p, e, st);
}

template <typename T, int D>
static int dkdv_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const unsigned grid = (unsigned)((p.N + 127) / 128) * (unsigned)(p.B * p.H * p.S);
    if (p.bias_dtype == EVO_NONE) mfma_dkdv<T, D, 0><<<grid, 256, 0, st>>>(p, e);
    else if (p.bias_dtype == EVO_F32) mfma_dkdv<T, D, 1><<<grid, 256, 0, st>>>(p, e);
    else mfma_dkdv<T, D, 2><<<grid, 256, 0, st>>>(p, e);
    return hip_rc();
}

int EVO_CAT(launch_mfma_delta_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int64_t rows = (int64_t)p.B * p.H * p.S * p.N;
    const unsigned grid = (unsigned)((rows + 255) / 256);
    if (p.dtype == EVO_BF16) mfma_delta<bf16_t, EVO_D><<<grid, 256, 0, st>>>(p, e.delta);
    else mfma_delta<f16_t, EVO_D><<<grid, 256, 0, st>>>(p, e.delta);
    return hip_rc();
}

int EVO_CAT(launch_mfma_dq_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? dq_bias<bf16_t, EVO_D>(p, e, st) : dq_bias<f16_t, EVO_D>(p, e, st);
}

int EVO_CAT(launch_mfma_dkdv_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? dkdv_bias<bf16_t, EVO_D>(p, e, st) : dkdv_bias<f16_t, EVO_D>(p, e, st);
}

}  // namespace evo
