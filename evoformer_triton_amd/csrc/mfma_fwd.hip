// Flash-style forward for gfx950 on the bf16/fp16 32x32x16 matrix-core instruction.
// Compiled once per head dim (-DEVO_D=8|16|32|64).
//
// Replaces the reference's `_attn_fwd` / `_attn_fwd_inner` (evoformer.py:23-297): bias add
// and mask fused before the running max (:68-71), online softmax (:71-89), P cast to the
// input dtype before P.V (:84), LSE = m + log(l) and O = acc / l in the epilogue (:285-297).
//
// Tiling.  One workgroup = 4 waves = 128 query rows of one problem (b,h,s); each wave owns
// 32 query rows for the whole key loop.  Keys are staged 64 at a time through LDS: K
// row-major, V transposed.  The score tile is computed transposed, S^T = K Q^T, so that a
// lane owns ONE query (column) and 16 keys (registers): the row max and row sum are
// in-lane reductions plus a single exchange between the two lane groups, the rescale of
// O^T is a per-lane scalar, and the probability tile in accumulator layout is already the
// B operand of O^T = V^T P^T.
#include "common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

template <typename T, int D, int BIASK>
__global__ void __launch_bounds__(256) mfma_fwd(EvoAttnParams p, Extra e) {
    constexpr int BQ = 128, BKV = 64;
    constexpr int DK = D < 16 ? 16 : D;  // contraction width of K Q^T, zero padded
    constexpr int KS = DK / 16;
    constexpr int DT = (D + 31) / 32;    // 32-row tiles of O^T
    constexpr int DP = DT * 32;
    constexpr int KP = DK + 8;           // LDS pitches, padded against bank conflicts
    constexpr int VP = BKV + 8;
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v2 v2;

    __shared__ __attribute__((aligned(16))) T Ks[BKV * KP];
    __shared__ __attribute__((aligned(16))) T Vt[DP * VP];
    __shared__ __attribute__((aligned(16))) float Ms[BKV];
    __shared__ float red[4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, g = lane >> 5;
    const int nqb = (p.N + BQ - 1) / BQ;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const unsigned pid = lid / nqb;
    const int q0 = (lid % nqb) * BQ + wave * 32;
    const Prob pr = decode_problem(p, pid);
    const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
    const int64_t sn = p.stride_n;
    const bool active = q0 < p.N;  // wave-uniform

    // zero the LDS padding that is read but never staged (d >= D)
    for (int i = tid; i < BKV * KP; i += 256) Ks[i] = (T)0.0f;
    for (int i = tid; i < DP * VP; i += 256) Vt[i] = (T)0.0f;

    // per-problem mask shift
    float shift = 0.0f;
    if (p.mask_kind != EVO_MASK_NONE) {
        float mx = -INFINITY;
        for (int j = tid; j < p.N; j += 256) mx = fmaxf(mx, mask_add(p, pr.b, pr.s, j));
        mx = wave_max(mx);
        if (lane == 0) red[wave] = mx;
        __syncthreads();
        shift = shift_from_max(fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
    }

    const int qrow = min(q0 + li, p.N - 1);
    v8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = ks * 16 + g * 8;
        qf[ks] = d0 < D ? ld8(Q + (int64_t)qrow * sn + d0) : zero8<T>();
    }
    const int64_t brow = (int64_t)pr.b * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h + (int64_t)qrow * p.bias_stride_row;
    const bool vec = e.vec_ok != 0;
    const float scale = p.scale;

    float m = -INFINITY, l = 0.0f;
    f32x16 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;

    for (int kv0 = 0; kv0 < p.N; kv0 += BKV) {
        __syncthreads();  // readers of the previous stage are done
        for (int it = tid; it < BKV * (D / 8); it += 256) {
            const int key = it / (D / 8), c = it % (D / 8), kk = kv0 + key;
            v8 val = kk < p.N ? ld8(K + (int64_t)kk * sn + c * 8) : zero8<T>();
            *reinterpret_cast<v8 *>(&Ks[key * KP + c * 8]) = val;
        }
        for (int it = tid; it < (BKV / 2) * (D / 8); it += 256) {
            const int jp = it / (D / 8), c = it % (D / 8), k0 = kv0 + 2 * jp;
            v8 a = k0 < p.N ? ld8(V + (int64_t)k0 * sn + c * 8) : zero8<T>();
            v8 b = k0 + 1 < p.N ? ld8(V + (int64_t)(k0 + 1) * sn + c * 8) : zero8<T>();
            const int pos = perm_pos(2 * jp);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v2 w;
                w[0] = a[i];
                w[1] = b[i];
                *reinterpret_cast<v2 *>(&Vt[(c * 8 + i) * VP + pos]) = w;
            }
        }
        if (tid < BKV) Ms[tid] = mask_add(p, pr.b, pr.s, kv0 + tid);
        __syncthreads();

        if (active) {
#pragma unroll
            for (int kt = 0; kt < BKV / 32; ++kt) {
                const int kb = kt * 32;
                if (kv0 + kb >= p.N) break;
                f32x16 acc;
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    v8 a = *reinterpret_cast<const v8 *>(&Ks[(kb + li) * KP + ks * 16 + g * 8]);
                    acc = Mfma<T>::mma(a, qf[ks], acc);
                }
                float t[16];
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int kl = kb + 8 * rr + 4 * g, kg = kv0 + kl;
                    float bv[4];
                    load_bias4<BIASK, T>(p.bias, brow + kg, p.N - kg, vec, bv);
                    const f32x4 mk = *reinterpret_cast<const f32x4 *>(&Ms[kl]);
#pragma unroll
                    for (int i = 0; i < 4; ++i) t[4 * rr + i] = fmaf(acc[4 * rr + i], scale, bv[i]) + mk[i];
                }
                if (shift != 0.0f) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) t[r] -= shift;
                }
                float mloc = t[0];
#pragma unroll
                for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, t[r]);
                mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
                const float mn = fmaxf(fmaxf(m, mloc), -FLT_MAX);
                const float alpha = fast_exp2((m - mn) * kLog2e);
                float pv[16], psum = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    pv[r] = fast_exp2((t[r] - mn) * kLog2e);
                    psum += pv[r];
                }
                l = l * alpha + psum;
                m = mn;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
#pragma unroll
                for (int ts = 0; ts < 2; ++ts) {
                    v8 pf;
#pragma unroll
                    for (int i = 0; i < 8; ++i) pf[i] = (T)pv[8 * ts + i];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        v8 a = *reinterpret_cast<const v8 *>(&Vt[(dt * 32 + li) * VP + kb + ts * 16 + g * 8]);
                        oacc[dt] = Mfma<T>::mma(a, pf, oacc[dt]);
                    }
                }
            }
        }
    }

    if (active) {
        l += __shfl_xor(l, 32);
        const float inv = 1.0f / l;
        const int q = q0 + li;
        if (q < p.N) {
            T *O = (T *)p.o + pr.base + (int64_t)q * sn;
            if (g == 0) p.lse[pr.row0 + q] = m + __logf(l);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const int d0 = dt * 32 + 8 * rr + 4 * g;
                    if (d0 < D)
                        store4<T>(O + d0, oacc[dt][4 * rr] * inv, oacc[dt][4 * rr + 1] * inv,
                                  oacc[dt][4 * rr + 2] * inv, oacc[dt][4 * rr + 3] * inv);
                }
        }
    }
}

template <typename T, int D>
static int fwd_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const unsigned nqb = (p.N + 127) / 128, grid = nqb * (unsigned)(p.B * p.H * p.S);
    if (p.bias_dtype == EVO_NONE) mfma_fwd<T, D, 0><<<grid, 256, 0, st>>>(p, e);
    else if (p.bias_dtype == EVO_F32) mfma_fwd<T, D, 1><<<grid, 256, 0, st>>>(p, e);
    else mfma_fwd<T, D, 2><<<grid, 256, 0, st>>>(p, e);
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

int EVO_CAT(launch_mfma_fwd_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? fwd_bias<bf16_t, EVO_D>(p, e, st) : fwd_bias<f16_t, EVO_D>(p, e, st);
}

}  // namespace evo
