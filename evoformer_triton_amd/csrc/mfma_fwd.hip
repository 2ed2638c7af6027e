// Flash-style forward for gfx950 on the bf16/fp16 32x32x16 matrix-core instruction.
// Compiled once per head dim (-DEVO_D=8|16|32|64).
//
// Replaces the reference's `_attn_fwd` / `_attn_fwd_inner` (evoformer.py:23-297): bias add
// and mask fused before the running max (:68-71), online softmax (:71-89), P cast to the
// input dtype before P.V (:84), LSE = m + log(l) and O = acc / l in the epilogue (:285-297).
//
// Tiling.  One workgroup = NW (4 or 8) waves = NW*32 query rows of one problem (b,h,s); each
// wave owns 32 query rows for the whole key loop.  Keys are staged up to 256 at a time through LDS: K
// row-major, V transposed.  The score tile is computed transposed, S^T = K Q^T, so that a
// lane owns ONE query (column) and 16 keys (registers): the row max and row sum are
// in-lane reductions plus a single exchange between the two lane groups, the rescale of
// O^T is a per-lane scalar, and the probability tile in accumulator layout is already the
// B operand of O^T = V^T P^T.
//
// The vector ALU, not the matrix core, bounds this kernel (one exp per score), so every
// addition that can be moved into the matmul is: Q is pre-multiplied by scale*log2(e), the
// bias tile (in log2 units and accumulator order, see prep.hip) is the C operand of the
// score MFMA, the mask rides along as three extra columns of K against ones in Q, and the
// running maximum as three more columns of Q against ones in K, so that after a problem's
// first 64 keys the scores arrive relative to it.  What is left per score is exp2, an
// addition and half a conversion; the maximum is searched, and the step rescaled, only in
// the first step and when a later step's sums show that its maximum moved far.
#include <type_traits>

#include "bwd_common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

// BT: 0 no bias; 1 fp32 tiles (times log2 e) or, for very few S rows, the caller's rows; 2 the
// tiles of a bias in the dtype of q as given (half the bytes per tile, 8 registers in flight
// instead of 16; unpacked and multiplied by log2 e right before they are used)
template <typename T, int D, int BT, int NW>
__global__ void __launch_bounds__(NW * 64, D >= 64 ? 2 : NW == 8 ? 4 : 3) mfma_fwd(EvoAttnParams p, Extra e) {
    constexpr bool HAS_BIAS = BT != 0, TILE16 = BT == 2;
    typedef typename std::conditional<TILE16, Tile16, f32x16>::type CTile;   // a bias tile on its way
    // The softmax that skips the search for the maximum after a problem's first 64 keys keeps a
    // second copy of the score code for the rare step that has to be redone; with fp32 bias
    // tiles in flight that does not fit 128 registers (8 waves) or 256 at head dim 128, and in
    // the 4-wave forms it measured no better on balance (B = 4, S = 1, H = 32, D = 64, fp32 bias
    // read from the caller's rows: N = 1024 136 against 130 TFLOP/s, N = 768 107 against 130):
    // the forms with an fp32 bias keep the plain online softmax, and so do head dims 64 and 128
    // (no bias, B = 4, S = 1, H = 32, D = 64, N = 1024: 72 against 62 us).
    constexpr bool LAZY = BT != 1 && D <= 32;
    constexpr int NTH = NW * 64;                  // threads per workgroup
    constexpr int BQ = NW * 32;                   // query rows per workgroup
    constexpr int BKV = D <= 32 ? 256 : 128;      // keys staged per round
    constexpr int SPS = BKV / 64;                 // 64-key steps per stage
    constexpr bool AUG_IN_PAD = D == 8;           // mask columns fit the zero padding of k-step 0
    constexpr int KW = AUG_IN_PAD ? 16 : D + 16;  // K row: data, 3 mask columns, zeros
    constexpr int KS = KW / 16;
    constexpr int AUGC = AUG_IN_PAD ? 8 : D;
    constexpr int DT = (D + 31) / 32;             // 32-row tiles of O^T
    constexpr int DP = DT * 32;
    constexpr int KP = KW + 8;                    // LDS pitches: conflict-free 16-byte reads
    constexpr int VP = BKV + 8;
    constexpr float TAU = 8.0f;                   // rescale only when the max grows by > 2^TAU
    // Q * scale * log2(e) is rounded to 16 bits; where the matrix core has k-steps to spare
    // (small head dims) the rounding residue rides along as a second operand, which makes
    // the scores exact to fp32.
    constexpr bool RESID = D <= 16;
    constexpr int KSD = (D + 15) / 16;
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v2 v2;

    __shared__ __attribute__((aligned(16))) T Ks[BKV * KP];
    __shared__ __attribute__((aligned(16))) T Vt[DP * VP];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: what depends on it branches and is addressed by the scalar unit
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32, npad = NT * 32;
    const int nqb = (p.N + BQ - 1) / BQ;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const unsigned pid = lid / nqb;
    const int q0 = (lid % nqb) * BQ + wave * 32;
    const Prob pr = walk_problem(p, pid);
    const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
    const int64_t sn = p.stride_n;
    const bool active = q0 < p.N;  // wave-uniform
    const int np256 = (p.N + 255) / 256 * 256;
    const uint4 *m2arow = e.m2a + ((int64_t)pr.b * p.S + pr.s) * np256;
    const bool dead = e.dead[pr.b * p.S + pr.s] != 0;

    // LDS that is read but never staged: the upper half of the mask k-step of K, rows d >= D
    // of V^T
    if (!AUG_IN_PAD)
        for (int key = tid; key < BKV; key += NTH)
            *reinterpret_cast<v8 *>(&Ks[key * KP + AUGC + 8]) = zero8<T>();
    if (DP > D)
        for (int i = tid; i < (DP - D) * VP / 8; i += NTH)
            *reinterpret_cast<v8 *>(&Vt[D * VP + i * 8]) = zero8<T>();

    // Q operand: data pre-multiplied by scale*log2(e); ones against the mask columns
    const int qrow = min(q0 + li, p.N - 1);
    const float c = p.scale * kLog2e;
    v8 qf[KS], qlo[KSD];
#pragma unroll
    for (int ks = 0; ks < KSD; ++ks) qlo[ks] = zero8<T>();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = ks * 16 + g * 8;
        qf[ks] = zero8<T>();
        if (d0 < D) {
            if (!dead) scaled_hilo8<T>(ld8(Q + (int64_t)qrow * sn + d0), c, qf[ks], qlo[ks < KSD ? ks : 0]);
        } else if (d0 == AUGC) {
            qf[ks][0] = qf[ks][1] = qf[ks][2] = (T)1.0f;
        }
    }

    // bias tiles of this wave's query rows; a dead problem reads the all-zero tile instead
    const int bb = e.bias_batches > 1 ? pr.b : 0;
    const int qt = min(q0 >> 5, NT - 1);
    const float *btile = dead ? e.bq + e.zero_tile + lane * 16
                              : e.bq + ((((int64_t)bb * p.H + pr.h) * NT + qt) * NT) * 1024 + lane * 16;
    const int64_t bstep = dead ? 0 : 1024;
    // or, for a bias that is used too few times to pay for the tiles, this lane's row of the
    // caller's tensor
    const bool bdirect = HAS_BIAS && e.bias_direct;
    const bool bf32 = p.bias_dtype == EVO_F32;
    const char *brow = (const char *)p.bias + ((int64_t)bb * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h +
                                               (int64_t)qrow * p.bias_stride_row) * (bf32 ? 4 : 2);
    const float bmul = dead ? 0.0f : kLog2e;
    const unsigned short *btile16 = !TILE16 ? nullptr
                                    : dead  ? e.bq16 + e.zero_tile + lane * 16
                                            : e.bq16 + ((((int64_t)bb * p.H + pr.h) * NT + qt) * NT) * 1024 + lane * 16;

    float m = LAZY ? 0.0f : -INFINITY, mf = 0.0f, l = 0.0f;
    f32x16 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;

    // Bias tile kt into 16 registers; past the last tile the previous one is read again
    // (every key there carries the mask floor, so the values do not matter).
    auto load_btile = [&](int kt, CTile &dst) {
        if constexpr (TILE16) {
            load_tile16(btile16 + (int64_t)min(kt, NT - 1) * bstep, dst);
        } else if (HAS_BIAS && bdirect) {   // uniform
            if (bf32) bias_tile_rows<T, true>(brow, min(kt, NT - 1) * 32, p.N, g, bmul, dst);
            else bias_tile_rows<T, false>(brow, min(kt, NT - 1) * 32, p.N, g, bmul, dst);
        } else if (HAS_BIAS) {
            const float *src = btile + (int64_t)min(kt, NT - 1) * bstep;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(src + 4 * rr);
                dst[4 * rr] = v[0]; dst[4 * rr + 1] = v[1]; dst[4 * rr + 2] = v[2]; dst[4 * rr + 3] = v[3];
            }
        }
    };

    // K and V rows are buffer loads: a resource (in scalar registers) that describes the problem's K or V rows and a
    // 32-bit byte offset per lane.  Rows at or beyond N lie past the end of the resource and read as zero (such keys
    // carry the mask floor), so no lane tests its row, and no 64-bit address per lane lives across the stages.
    const int kv_valid = (int)(((int64_t)(p.N - 1) * sn + D) * 2);   // bytes from the first K (V) row to the end of the last
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc((void *)K, 0, kv_valid, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc((void *)V, 0, kv_valid, 0x00020000);
    const int sn2 = (int)sn * 2;
    auto stage = [&](int kv0) {
        __syncthreads();  // readers of the previous stage are done
        for (int it = tid; it < BKV * (D / 8); it += NTH) {
            const int key = it / (D / 8), ch = it % (D / 8), kk = kv0 + key;
            const v8 val = __builtin_bit_cast(v8, __builtin_amdgcn_raw_buffer_load_b128(krs, kk * sn2 + ch * 16, 0, 0));
            *reinterpret_cast<v8 *>(&Ks[key * KP + ch * 8]) = val;
        }
        for (int key = tid; key < BKV; key += NTH)   // (mask hi, mid, lo, 1, 1, 1, 0, 0); the floor past the padded N
            *reinterpret_cast<uint4 *>(&Ks[key * KP + AUGC]) = m2arow[min(kv0 + key, np256 - 1)];
        constexpr int NPAIR = BKV / 2;
        for (int it = tid; it < NPAIR * (D / 8); it += NTH) {
            const int ch = it / NPAIR, jp = it % NPAIR, k0 = kv0 + 2 * jp;
            const v8 a = __builtin_bit_cast(v8, __builtin_amdgcn_raw_buffer_load_b128(vrs, k0 * sn2 + ch * 16, 0, 0));
            const v8 b = __builtin_bit_cast(v8, __builtin_amdgcn_raw_buffer_load_b128(vrs, (k0 + 1) * sn2 + ch * 16, 0, 0));
            const int pos = perm_pos(2 * jp);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v2 w;
                w[0] = a[i];
                w[1] = b[i];
                *reinterpret_cast<v2 *>(&Vt[(ch * 8 + i) * VP + pos]) = w;
            }
        }
        __syncthreads();
    };

    // One 64-key step: two score tiles, online softmax, four P.V k-steps.  The bias tiles
    // c0, c1 are consumed by the first score MFMAs; the same registers then receive the
    // tiles of the next step, which travel while the softmax and P.V run.
    auto cval = [&](const CTile &t) -> f32x16 {
        if constexpr (!HAS_BIAS) {
            f32x16 z;
#pragma unroll
            for (int r = 0; r < 16; ++r) z[r] = 0.0f;
            return z;
        } else if constexpr (TILE16) {
            f32x16 v;
            unpack_tile16<T>(t, bmul, v);
            return v;
        } else {
            return t;
        }
    };
    // m is the maximum the probabilities are relative to, mf what the mask k-step subtracts
    // inside the MFMA (m, or 0 while m is unknown or too large to be carried in three 16-bit
    // columns next to scores of order one): after a problem's first 64 keys the scores leave
    // the matrix core relative to m and the common step neither searches its maximum nor
    // subtracts.
    // one 32-key score tile (keys kb .. kb + 31 of the stage) on top of its bias tile
    auto score1 = [&](int kb, const f32x16 &bias, f32x16 &a) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            v8 k = *reinterpret_cast<const v8 *>(&Ks[(kb + li) * KP + ks * 16 + g * 8]);
            a = Mfma<T>::mma(k, qf[ks], ks == 0 ? bias : a);
            if (RESID && ks < KSD) a = Mfma<T>::mma(k, qlo[ks], a);
        }
    };
    // where the maximum stands; `used` is the mf the step's scores were formed with
    auto settle = [&](bool first, f32x16 &a0, f32x16 &a1, float used) {
        float mloc = fmaxf(a0[0], a1[0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, fmaxf(a0[r], a1[r]));
        {   // exchange between the two lane groups without touching LDS
            const unsigned u = __float_as_uint(mloc);
            auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
            mloc = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
        }
        const float cand = mloc + used;
        // move m only when the maximum grows by more than 2^TAU (always at the first step)
        const bool grow = first || cand > m + TAU;
        if (__any(grow || m != used)) {
            const float mn = grow ? cand : m;
            if (!first) {
                const float alpha = fast_exp2(m - mn);   // <= 1; 1 where this lane's m stays
                l *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
            }
            m = mn;
            const float dsub = m - used;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                a0[r] -= dsub;
                a1[r] -= dsub;
            }
            // from the next scores on the MFMA subtracts m itself
            mf = fabsf(m) <= 1024.0f ? m : 0.0f;
            const v8 qa = aug8<T>(ones3<T>(), pack_split3<T>(-mf));   // ones x mask columns, -mf x ones
            if (g == (AUG_IN_PAD ? 1 : 0)) qf[KS - 1] = qa;
        }
    };
    // P = exp2 and this lane's sum of them in fp32 (the reference sums before it rounds,
    // evoformer.py:77-84: the log-sum-exp the backward normalises with carries no rounding of
    // P, which on a peaked row would be a relative 2^-9 on every gradient), then P rounded to T
    auto probs = [&](f32x16 &a0, f32x16 &a1, v8 (&pf)[4], float &ls) {
        ls = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            a0[r] = fast_exp2(a0[r]);
            a1[r] = fast_exp2(a1[r]);
            ls += a0[r] + a1[r];
        }
#pragma unroll
        for (int ts = 0; ts < 4; ++ts)
#pragma unroll
            for (int i = 0; i < 8; ++i) pf[ts][i] = (T)((ts < 2 ? a0 : a1)[8 * (ts & 1) + i]);
    };
    auto compute = [&](int step, CTile &c0, CTile &c1) {
        const int kb = (step % SPS) * 64;
        const float used = mf;
        f32x16 a0, a1;
        score1(kb, cval(c0), a0);
        score1(kb + 32, cval(c1), a1);
        load_btile(2 * step + 2, c0);
        load_btile(2 * step + 3, c1);
        if constexpr (!LAZY) {
            // the plain online softmax: maximum of every step, subtraction, fp32 row sums
            float mloc = fmaxf(a0[0], a1[0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, fmaxf(a0[r], a1[r]));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
            const bool grow = mloc > m + TAU;
            if (__any(grow)) {
                const float mn = grow ? mloc : m;
                const float alpha = fast_exp2(m - mn);
                l *= alpha;
                m = mn;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
            }
            float psum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                a0[r] = fast_exp2(a0[r] - m);
                a1[r] = fast_exp2(a1[r] - m);
                psum += a0[r] + a1[r];
            }
            l += psum;
#pragma unroll
            for (int ts = 0; ts < 4; ++ts) {
                v8 pf1;
#pragma unroll
                for (int i = 0; i < 8; ++i) pf1[i] = (T)((ts < 2 ? a0 : a1)[8 * (ts & 1) + i]);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    v8 va = *reinterpret_cast<const v8 *>(&Vt[(dt * 32 + li) * VP + kb + ts * 16 + g * 8]);
                    oacc[dt] = Mfma<T>::mma(va, pf1, oacc[dt]);
                }
            }
            return;
        }
        v8 pf[4];
        float ls;
        const bool lazy = step != 0 && !__any(m != used);
        if (!lazy) settle(step == 0, a0, a1, used);
        probs(a0, a1, pf, ls);
        // A lane sum beyond 2^13 (or not a number) means some score stands far above m: the step
        // is then redone the long way, from the bias tiles read again.
        if (__builtin_expect(lazy && __any(!(ls <= 8192.0f)), 0)) {
            CTile t;
            load_btile(2 * step, t);
            score1(kb, cval(t), a0);
            load_btile(2 * step + 1, t);
            score1(kb + 32, cval(t), a1);
            settle(false, a0, a1, used);
            probs(a0, a1, pf, ls);
        }
        l += ls;
#pragma unroll
        for (int ts = 0; ts < 4; ++ts) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                v8 va = *reinterpret_cast<const v8 *>(&Vt[(dt * 32 + li) * VP + kb + ts * 16 + g * 8]);
                oacc[dt] = Mfma<T>::mma(va, pf[ts], oacc[dt]);
            }
        }
    };

    const int nsteps = (p.N + 63) / 64;
    CTile c0, c1;
    load_btile(0, c0);
    load_btile(1, c1);
    for (int step = 0; step < nsteps; ++step) {
        if (step % SPS == 0) stage(step * 64);
        if (active) compute(step, c0, c1);
    }

    if (active) {
        l += __shfl_xor(l, 32);
        const float inv = 1.0f / l;
        const int q = q0 + li;
        if (q < p.N) {
            T *O = (T *)p.o + pr.base + (int64_t)q * sn;
            // natural-log LSE of the (shifted) scores, as the reference stores it (:285-288)
            if (g == 0) p.lse[pr.row0 + q] = (m + __log2f(l)) * kLn2;
            if (p.o) {   // uniform (with a gate the caller may ask for the gated output alone)
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
            if (p.gate) {   // uniform: sigmoid(gate) * O goes out as a second tensor, from the same registers
                const int64_t off = pr.base + (int64_t)q * sn;
                T *Og = (T *)p.o_gated + off;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[dt][r] *= inv;
                    gate_row_tile<T>((const T *)p.gate + off, dt * 32, D, oacc[dt], g);
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const int d0 = dt * 32 + 8 * rr + 4 * g;
                        if (d0 < D)
                            store4<T>(Og + d0, oacc[dt][4 * rr], oacc[dt][4 * rr + 1], oacc[dt][4 * rr + 2], oacc[dt][4 * rr + 3]);
                    }
                }
            }
        }
    }
}

template <typename T, int D, int NW>
static int fwd_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const unsigned nqb = (p.N + NW * 32 - 1) / (NW * 32), grid = nqb * (unsigned)(p.B * p.H * p.S);
    if (p.bias_dtype == EVO_NONE) mfma_fwd<T, D, 0, NW><<<grid, NW * 64, 0, st>>>(p, e);
    else if (e.bq16 && !e.bias_direct) mfma_fwd<T, D, 2, NW><<<grid, NW * 64, 0, st>>>(p, e);
    else mfma_fwd<T, D, 1, NW><<<grid, NW * 64, 0, st>>>(p, e);
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

// 8 waves (256 query rows) per workgroup stage K and V once for twice the rows; worth it
// unless the last workgroup of a problem would be more than half empty.
template <typename T, int D>
static int fwd_waves(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int rem = p.N % 256;
    bool wide = p.N >= 256 && (rem == 0 || rem > 128);
    // ... and unless there are too few problems for that: below four workgroups per CU (256
    // CUs) the narrower form's twice as many workgroups fill the chip better (the reference's
    // speed benchmark has 128 problems).  EVO_FLAG_DEBUG_OTHER_WIDTH inverts the choice, for comparison.
    const int64_t wgs = (int64_t)((p.N + 255) / 256) * p.B * p.H * p.S;
    if (wgs < 1024) wide = false;
    if (p.flags & EVO_FLAG_DEBUG_OTHER_WIDTH) wide = !wide;
    return wide ? fwd_bias<T, D, 8>(p, e, st) : fwd_bias<T, D, 4>(p, e, st);
}

int EVO_CAT(launch_mfma_fwd_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? fwd_waves<bf16_t, EVO_D>(p, e, st) : fwd_waves<f16_t, EVO_D>(p, e, st);
}

}  // namespace evo
