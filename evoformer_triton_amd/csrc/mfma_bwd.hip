// Backward kernels for gfx950 on the bf16/fp16 32x32x16 matrix-core instruction.
// Compiled once per head dim (-DEVO_D=8|16|32|64).
//
// They replace the reference's `_attn_bwd_preprocess` (evoformer.py:299-326),
// `_attn_bwd_dq` (:329-476) and `_attn_bwd_dk_dv` (:479-630).  Both kernels recompute
// P = exp(score - LSE) from the saved log-sum-exp (:452, :600), form
// dS = P * (dP - delta) (:456, :610) and cast P and dS to the input dtype before the
// gradient matmuls (:459, :603, :611); dQ and dK are multiplied by the softmax scale after
// the matmul (:462, :614).
//
// As in the forward, the vector ALU is the scarce unit (one exp per score, twice), so every
// addition is folded into the matrix core: one operand is pre-multiplied by
// scale*log2(e), the bias tile (log2 units, accumulator order, see prep.hip) is the C
// operand of the score MFMA, and mask, -LSE and -delta travel as three 16-bit columns
// each (hi + mid + lo, exact to 24 bits) in one extra k-step against columns of ones.
// The score MFMA then yields log2 P directly and the dO.V^T MFMA yields dP - delta; per
// score there remain exp2, one multiply and the two conversions.
//
// dBias is the sum of dS over S.  The reference adds every fp32 dS tile into global memory
// with atomics (:458).  Here the dQ kernel owns a 32-query slab of one head for a whole
// chunk of S rows and keeps the running sum of dS for that slab in registers (fp32
// additions of the fp32 dS, as the reference adds fp32 dS at :456-459), writes one partial
// per chunk, and a second kernel adds the partials in a fixed order: no floating-point
// atomics, bit-reproducible.
#include <type_traits>

#include "bwd_common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

// ------------------------------------------------------------------ dQ, delta and dBias partials
//
// Workgroup = 4 waves = (b, h, chunk of S, 32 query rows).  The waves split the keys:
// wave w takes 32-key tiles w, w+4, w+8, ...  Scores are computed transposed
// (S^T = K Q^T, dP^T = V dO^T) so that a lane owns one query and 16 keys, which makes the
// dS^T accumulator tile the B operand of dQ^T += K^T dS^T and lines up with the dBias^T sums.
// Each wave's partial dQ^T meets the others in LDS once per S row and is summed in wave
// order.  Query slab and head are fixed for the whole S loop, so for N <= 512 the bias
// tiles stay in registers across it.  delta = rowsum(dO * O) (evoformer.py:313-323) is
// formed here from the rows the kernel loads anyway and written out for the dK/dV kernel.
template <typename T, int D, bool HAS_BIAS, int NTW>
__global__ void __launch_bounds__(256) mfma_dq(EvoAttnParams p, Extra e) {
    typedef Geo<D> G;
    constexpr int KS = G::KS, KSD = G::KSD, DT = G::DT, DP = G::DP, AUGC = G::AUGC;
    constexpr int RP = DT * 32 + 4;   // pitch of a partial dQ row in LDS (floats)
    constexpr int KTP = 32 + 8;       // pitch of a transposed K tile row
    constexpr bool BIAS_RESIDENT = HAS_BIAS && NTW <= 4;
    constexpr int NRES = BIAS_RESIDENT ? NTW : 1;
    typedef typename Mfma<T>::v8 v8;

    __shared__ __attribute__((aligned(16))) float red[4 * 32 * RP];
    __shared__ __attribute__((aligned(16))) T Kt[4 * DP * KTP];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: what depends on it branches and is addressed by the scalar unit
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32, npad = NT * 32;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const int qt = lid % NT;
    const unsigned bh = (lid / NT) % (unsigned)(p.B * p.H);
    const int c = lid / NT / (unsigned)(p.B * p.H);
    const int b = bh / p.H, h = bh % p.H;
    const int q0 = qt * 32;
    const int qrow = min(q0 + li, p.N - 1);
    const int64_t sn = p.stride_n;
    const bool want_dbias = e.dbias_part != nullptr && p.dbias != nullptr;
    const float cs = p.scale * kLog2e;
    T *Ktw = Kt + wave * DP * KTP;

    // rows d >= D of the transposed K tile are read by the MFMA but never written
    if (DP > D)
        for (int i = lane; i < (DP - D) * KTP; i += 64) Ktw[D * KTP + i] = (T)0.0f;

    f32x16 dbacc[NTW];
#pragma unroll
    for (int j = 0; j < NTW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) dbacc[j][r] = 0.0f;

    const int bb = e.bias_batches > 1 ? b : 0;
    const int64_t tile0 = ((((int64_t)bb * p.H + h) * NT + qt) * NT) * 1024;
    const float *btile0 = e.bq + tile0 + lane * 16;
    const float *ztile = e.bq + e.zero_tile + lane * 16;
    // or, for a bias that is used too few times to pay for the tiles, this lane's row of the
    // caller's tensor
    const bool bdirect = HAS_BIAS && e.bias_direct;
    const bool bf32 = p.bias_dtype == EVO_F32;
    const char *brow = (const char *)p.bias + ((int64_t)bb * p.bias_stride_b + (int64_t)h * p.bias_stride_h +
                                               (int64_t)qrow * p.bias_stride_row) * (bf32 ? 4 : 2);
    // key tile kt of this wave's query rows, in log2 units (zero for a row with every key masked)
    auto load_btile = [&](int kt, bool dead_row, f32x16 &dst) {
        if (bdirect) {   // uniform
            const float mul = dead_row ? 0.0f : kLog2e;
            if (bf32) bias_tile_rows<T, true>(brow, kt * 32, p.N, g, mul, dst);
            else bias_tile_rows<T, false>(brow, kt * 32, p.N, g, mul, dst);
            return;
        }
        if (e.bq16) {   // uniform: a bias in the dtype of q is prepared as given, 16 bits per entry
            Tile16 t;
            load_tile16(e.bq16 + (dead_row ? e.zero_tile : tile0 + (int64_t)kt * 1024) + lane * 16, t);
            unpack_tile16<T>(t, dead_row ? 0.0f : kLog2e, dst);
            return;
        }
        const float *src = dead_row ? ztile : btile0 + (int64_t)kt * 1024;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(src + 4 * rr);
            dst[4 * rr] = v[0]; dst[4 * rr + 1] = v[1]; dst[4 * rr + 2] = v[2]; dst[4 * rr + 3] = v[3];
        }
    };
    f32x16 bres[NRES];
    if (BIAS_RESIDENT) {
#pragma unroll
        for (int j = 0; j < NRES; ++j) load_btile(min(wave + 4 * j, NT - 1), false, bres[j]);
    }

    const uint2 one3 = ones3<T>();
    const uint2 zero3 = {0u, 0u};
    const int s_begin = c * e.chunk, s_end = min(p.S, s_begin + e.chunk);
    for (int s = s_begin; s < s_end; ++s) {
        const unsigned pid = (bh * (unsigned)p.S) + s;
        const Prob pr = decode_problem(p, pid);
        const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
        const T *Gd = (const T *)p.dout + pr.base;
        // (where delta is given, by the gate's pass, there may be no ungated O: the loads go to dO instead and their sum is dropped)
        const T *O = e.delta_given ? Gd : (const T *)p.o + pr.base;
        const uint2 *m2row = e.m2 + ((int64_t)b * p.S + s) * npad;
        const bool dead = e.dead[b * p.S + s] != 0;
        const bool kill = dead && p.mask_kind == EVO_MASK_BOOL;

        // this lane's half of the query row: Q (scaled), dO, and delta = <dO, O>
        v8 qf[KS], gf[KS], qlo[KSD];
        float dpart = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KSD; ++ks) qlo[ks] = zero8<T>();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 16 + g * 8;
            qf[ks] = zero8<T>();
            gf[ks] = zero8<T>();
            if (d0 < D) {
                v8 qraw = ld8(Q + (int64_t)qrow * sn + d0);
                gf[ks] = ld8(Gd + (int64_t)qrow * sn + d0);
                v8 oraw = ld8(O + (int64_t)qrow * sn + d0);
                if (!dead) scaled_hilo8<T>(qraw, cs, qf[ks], qlo[ks < KSD ? ks : 0]);
                dpart = dot8<T>(gf[ks], oraw, dpart);
            }
        }
        const float dl = e.delta_given ? e.delta[pr.row0 + qrow] : dpart + __shfl_xor(dpart, 32);
        const float lse2 = p.lse[pr.row0 + qrow] * kLog2e;
        if (!e.delta_given && wave == 0 && g == 0 && q0 + li < p.N) e.delta[pr.row0 + q0 + li] = dl;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks * 16 + g * 8 == AUGC) {
                qf[ks] = aug8<T>(one3, pack_split3<T>(-lse2));   // ones x mask, -lse x ones
                gf[ks] = aug8<T>(pack_split3<T>(-dl), zero3);    // -delta x ones
            }
        }

        f32x16 dqacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dqacc[dt][r] = 0.0f;

#pragma unroll 1
        for (int j = 0; j < NTW; ++j) {
            const int kt = wave + 4 * j;
            if (kt < NT) {  // wave-uniform
                const int kb = kt * 32;
                const int keyc = min(kb + li, p.N - 1);
                v8 ka[KS], va[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int d0 = ks * 16 + g * 8;
                    ka[ks] = zero8<T>();
                    va[ks] = zero8<T>();
                    if (d0 < D) {
                        ka[ks] = ld8(K + (int64_t)keyc * sn + d0);
                        va[ks] = ld8(V + (int64_t)keyc * sn + d0);
                    } else if (d0 == AUGC || G::aug_step(ks)) {  // (qf, gf are zero in the step's upper half)
                        ka[ks] = aug8<T>(m2row[kb + li], one3);  // mask x ones, ones x -lse
                        va[ks] = aug8<T>(one3, zero3);           // ones x -delta
                    }
                }
                // transposed copy of the K tile for dQ^T += K^T dS^T (wave-private LDS)
#pragma unroll
                for (int ks = 0; ks < KSD; ++ks) {
                    const int d0 = ks * 16 + g * 8;
                    if (d0 < D) {
#pragma unroll
                        for (int i = 0; i < 8; ++i) Ktw[(d0 + i) * KTP + perm_pos(li)] = ka[ks][i];
                    }
                }
                f32x16 acc, dp;
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = dp[r] = 0.0f;
                if (HAS_BIAS) {
                    if (BIAS_RESIDENT) {
                        // compare chain: a static register index for a run-time tile number
#pragma unroll
                        for (int jj = 0; jj < NRES; ++jj)
                            if (jj == j) acc = bres[jj];
                        if (dead) {
#pragma unroll
                            for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
                        }
                    } else {
                        load_btile(kt, dead, acc);
                    }
                }
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    acc = Mfma<T>::mma(ka[ks], qf[ks], acc);   // log2 P^T
                    if (G::RESID && ks < KSD) acc = Mfma<T>::mma(ka[ks], qlo[ks], acc);
                    dp = Mfma<T>::mma(va[ks], gf[ks], dp);     // dP^T - delta
                }
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) ds[r] = fast_exp2(acc[r]) * dp[r];
                if (kill) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) ds[r] = 0.0f;
                }
                if (want_dbias) {
                    // fp32 sums of the fp32 dS (compare chain: a static register index for a run-time tile number)
#pragma unroll
                    for (int jj = 0; jj < NTW; ++jj)
                        if (jj == j) {
#pragma unroll
                            for (int r = 0; r < 16; ++r) dbacc[jj][r] += ds[r];
                        }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int ts = 0; ts < 2; ++ts) {
                    v8 dsf;
#pragma unroll
                    for (int i = 0; i < 8; ++i) dsf[i] = (T)ds[8 * ts + i];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        v8 kta = *reinterpret_cast<const v8 *>(&Ktw[(dt * 32 + li) * KTP + ts * 16 + g * 8]);
                        dqacc[dt] = Mfma<T>::mma(kta, dsf, dqacc[dt]);
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
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
                store4<T>(dQ + (int64_t)(q0 + q) * sn + d4, sum[0] * p.scale, sum[1] * p.scale, sum[2] * p.scale,
                          sum[3] * p.scale);
        }
        __syncthreads();  // red is rewritten by the next S row
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
// Workgroup = NW (4 or 8) waves = NW*32 keys of one problem; each wave keeps its 32 keys' K and V
// operands in registers and loops over all query rows.  Those are staged in LDS once,
// row-major: Q pre-multiplied by scale*log2(e) exactly as in the forward, dO, and per query the
// 16-bit columns that carry -LSE and -delta into the score MFMAs.  The transposed operands
// of dV^T += dO^T P and dK^T += Q^T dS come from the same rows by transposing LDS reads
// (`ds_read_b64_tr_b16`).  Q is staged a second time as given: dK sums over that copy and is
// multiplied by scale at the end (summing over the rounded scaled Q alone costs dK two digits
// at N = 768); for head dims <= 16 the rounding residue of the scaled Q is staged as well, for
// the scores only (a third set of transposing reads and twice the dK MFMAs if dK used it).
// Scores are NOT transposed here: a lane owns one key and 16 queries, so that P and dS in
// accumulator layout are the B operands of the two gradient matmuls.
template <int D>
struct KvGeo {
    static constexpr int C = D / 8;                          // 16-byte chunks per row
    static constexpr int RPB = 16 / C > 0 ? 16 / C : 1;      // rows per 256 bytes
    static constexpr int BQS = D <= 32 ? 256 : 128;          // query rows staged per round
    static constexpr bool RESID = D <= 16;
    // LDS layout for `rows` staged query rows (BQS, or 128 where a problem has no more):
    //   [Q scaled][Q as given][dO]([rounding residue of Q scaled] for RESID)[-LSE columns][-delta columns]
    static __host__ __device__ constexpr int lds_bytes(int rows) { return rows * ((RESID ? 4 : 3) * D * 2 + 32); }
    static __device__ __forceinline__ int swz(int r, int c) { return r * (D * 2) + ((c ^ ((r / RPB) % C)) << 4); }
};

typedef short s16x4 __attribute__((ext_vector_type(4)));

#ifdef EVO_TRACE
#define EVO_TK(slot)                                                                             \
    do {                                                                                         \
        if (e.trace && (threadIdx.x & 63) == 0)                                                  \
            e.trace[((int64_t)blockIdx.x * 8 + (threadIdx.x >> 6)) * 16 + (slot)] = wall_clock64(); \
    } while (0)
#else
#define EVO_TK(slot) do {} while (0)
#endif

// BT: 0 no bias; 1 fp32 tiles (times log2 e) or, for very few S rows, the caller's columns; 2 the
// tiles of a bias in the dtype of q as given (half the bytes per tile, 8 registers in flight
// instead of 16; unpacked and multiplied by log2 e right before they are used)
template <typename T, int D, int BT, int NW, int ROWS>
__global__ void __launch_bounds__(NW * 64, D >= 64 ? 2 : NW == 8 ? 4 : 3) mfma_dkdv(EvoAttnParams p, Extra e) {
    typedef Geo<D> G;
    typedef KvGeo<D> R;
    constexpr bool HAS_BIAS = BT != 0, TILE16 = BT == 2;
    typedef typename std::conditional<TILE16, Tile16, f32x16>::type CTile;   // a bias tile on its way
    constexpr int KS = G::KS, KSD = G::KSD, DT = G::DT, AUGC = G::AUGC;
    constexpr int NTH = NW * 64;
    constexpr int BK = NW * 32;
    // the 8-wave form runs at 128 registers: prefetching a 16-register tile there spills (227 vs 187 us)
    constexpr bool PREFETCH = NW == 4 || TILE16;
    constexpr int BQS = ROWS, C = R::C;      // query rows staged per round
    constexpr int TPS = BQS / 32;            // query tiles per stage
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v4 v4;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    EVO_TK(0);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: what depends on it branches and is addressed by the scalar unit
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32, npad = NT * 32;
    const int nkb = (p.N + BK - 1) / BK;
    constexpr int srows = BQS;
    constexpr int BLK = srows * D * 2;
    constexpr int OFF_QS = 0, OFF_QR = BLK, OFF_G = 2 * BLK, OFF_QL = 3 * BLK;
    constexpr int OFF_AQ = (R::RESID ? 4 : 3) * BLK, OFF_AG = OFF_AQ + srows * 16;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const unsigned pid = lid / nkb;
    const int key0 = (lid % nkb) * BK + wave * 32;
    const Prob pr = walk_problem(p, pid);
    const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
    const T *Gd = (const T *)p.dout + pr.base;
    const int64_t sn = p.stride_n;
    const bool active = key0 < p.N;
    const int key = key0 + li, keyc = min(key, p.N - 1);
    const bool dead = e.dead[pr.b * p.S + pr.s] != 0;
    const bool kill = dead && p.mask_kind == EVO_MASK_BOOL;
    const bool want_dm = e.dmask_part != nullptr && p.dmask != nullptr;
    const float cs = p.scale * kLog2e;
    const uint2 one3 = ones3<T>();
    const uint2 zero3 = {0u, 0u};

    // (where the caller asks for it: the dBias partials summed on the way in, by the workgroups that start first)
    if (e.dbias_chunks > 0) sum_dbias_partials<NTH>(p, e, tid);

    // this wave's keys: requested now, used after the queries have been staged, so that the
    // two round trips to memory overlap
    v8 kraw[KSD], vraw[KSD];
#pragma unroll
    for (int ks = 0; ks < KSD; ++ks) {
        const int d0 = min(ks * 16 + g * 8, D - 8);
        kraw[ks] = ld8(K + (int64_t)keyc * sn + d0);
        vraw[ks] = ld8(V + (int64_t)keyc * sn + d0);
    }
    const uint2 mraw = e.m2[((int64_t)pr.b * p.S + pr.s) * npad + min(key, npad - 1)];
    v8 kf[KS], vf[KS], kres[KSD];   // the operands built from them

    const int bb = e.bias_batches > 1 ? pr.b : 0;
    const int ktc = min(key0 >> 5, NT - 1);
    const float *btile = dead ? e.bk + e.zero_tile + lane * 16
                              : e.bk + (((int64_t)bb * p.H + pr.h) * NT * NT + ktc) * 1024 + lane * 16;
    const int64_t bstep = dead ? 0 : (int64_t)NT * 1024;  // next query tile, same key tile
    // or, for a bias that is used too few times to pay for the tiles, this lane's column of
    // the caller's tensor
    const bool bdirect = HAS_BIAS && e.bias_direct;
    const bool bf32 = p.bias_dtype == EVO_F32;
    const char *bmat = (const char *)p.bias + ((int64_t)bb * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h) * (bf32 ? 4 : 2);
    const float bmul = dead ? 0.0f : kLog2e;
    const unsigned short *btile16 = !TILE16 ? nullptr
                                    : dead  ? e.bk16 + e.zero_tile + lane * 16
                                            : e.bk16 + (((int64_t)bb * p.H + pr.h) * NT * NT + ktc) * 1024 + lane * 16;
    auto cval = [&](const CTile &t) -> f32x16 {
        if constexpr (TILE16) {
            f32x16 v;
            unpack_tile16<T>(t, bmul, v);
            return v;
        } else {
            return t;
        }
    };
    auto load_btile = [&](int qt, CTile &dst) {
        if constexpr (TILE16) {
            load_tile16(btile16 + (int64_t)min(qt, NT - 1) * bstep, dst);
        } else if (HAS_BIAS && bdirect) {   // uniform
            if (bf32) bias_tile_cols<T, true>(bmat, keyc, min(qt, NT - 1) * 32, p.N, (unsigned)p.bias_stride_row, g, bmul, dst);
            else bias_tile_cols<T, false>(bmat, keyc, min(qt, NT - 1) * 32, p.N, (unsigned)p.bias_stride_row, g, bmul, dst);
        } else if (HAS_BIAS) {
            const float *src = btile + (int64_t)min(qt, NT - 1) * bstep;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(src + 4 * rr);
                dst[4 * rr] = v[0]; dst[4 * rr + 1] = v[1]; dst[4 * rr + 2] = v[2]; dst[4 * rr + 3] = v[3];
            }
        }
    };

    f32x16 dk[DT], dv[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dk[dt][r] = dv[dt][r] = 0.0f;
    float dm = 0.0f;

    const int row_valid = (int)(((int64_t)(p.N - 1) * sn + D) * 2);   // bytes from a problem's first row to the end of its last
    const __amdgpu_buffer_rsrc_t qrs = __builtin_amdgcn_make_buffer_rsrc((void *)Q, 0, row_valid, 0x00020000);
    const __amdgpu_buffer_rsrc_t grs = __builtin_amdgcn_make_buffer_rsrc((void *)Gd, 0, row_valid, 0x00020000);
    const int sn2 = (int)sn * 2;
    auto stage = [&](int qs0) {
        EVO_TK(1);
        __syncthreads();
        EVO_TK(2);
        // all loads first, then the conversions and LDS writes: one round trip, not one per piece
        constexpr int NIT = (srows * C + NTH - 1) / NTH;
        v8 qv[NIT], gv[NIT];
        // (buffer loads: 32-bit lane offsets from the problem's first row; a row at or beyond N lies past the end of
        // the resource and reads as zero)
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int it = tid + i * NTH;
            const int row = min(it / C, srows - 1), ch = it % C, off = (qs0 + row) * sn2 + ch * 16;
            qv[i] = __builtin_bit_cast(v8, __builtin_amdgcn_raw_buffer_load_b128(qrs, off, 0, 0));
            gv[i] = __builtin_bit_cast(v8, __builtin_amdgcn_raw_buffer_load_b128(grs, off, 0, 0));
        }
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int it = tid + i * NTH;
            if (it < srows * C) {
                const int row = it / C, ch = it % C;
                const v8 a = qv[i];
                const v8 bb2 = gv[i];
                // the score operand carries scale*log2(e), rounded exactly as in the forward
                v8 hi, lo;
                scaled_hilo8<T>(a, cs, hi, lo);
                const int o = R::swz(row, ch);
                *reinterpret_cast<v8 *>(lds + OFF_QS + o) = hi;
                *reinterpret_cast<v8 *>(lds + OFF_QR + o) = a;
                *reinterpret_cast<v8 *>(lds + OFF_G + o) = bb2;
                if (R::RESID) *reinterpret_cast<v8 *>(lds + OFF_QL + o) = lo;
            }
        }
        for (int row = tid; row < srows; row += NTH) {
            const int qq = qs0 + row;
            // rows past N get -LSE = floor: their probabilities vanish
            const float nl = qq < p.N ? -p.lse[pr.row0 + qq] * kLog2e : kMaskFloor;
            const float nd = qq < p.N ? -e.delta[pr.row0 + qq] : 0.0f;
            *reinterpret_cast<v8 *>(lds + OFF_AQ + row * 16) = aug8<T>(one3, pack_split3<T>(nl));
            *reinterpret_cast<v8 *>(lds + OFF_AG + row * 16) = aug8<T>(pack_split3<T>(nd), zero3);
        }
        EVO_TK(3);
        __syncthreads();
        EVO_TK(4);
    };

    // one 32-query tile against this wave's 32 keys
    auto compute = [&](int qtile, CTile &ctile) {
        const int qb = (qtile % TPS) * 32;
        f32x16 acc, dp;
#pragma unroll
        for (int r = 0; r < 16; ++r) dp[r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 16 + g * 8;
            v8 qa = zero8<T>(), ga = zero8<T>();
            if (d0 < D) {
                const int o = R::swz(qb + li, 2 * ks + g);
                qa = *reinterpret_cast<const v8 *>(lds + OFF_QS + o);
                ga = *reinterpret_cast<const v8 *>(lds + OFF_G + o);
            } else if (d0 == AUGC || G::aug_step(ks)) {   // (kf, vf are zero in the step's upper half)
                qa = *reinterpret_cast<const v8 *>(lds + OFF_AQ + (qb + li) * 16);
                ga = *reinterpret_cast<const v8 *>(lds + OFF_AG + (qb + li) * 16);
            }
            if (ks == 0) {
                if (HAS_BIAS) {
                    acc = Mfma<T>::mma(qa, kf[0], cval(ctile));
                } else {
                    f32x16 z;
#pragma unroll
                    for (int r = 0; r < 16; ++r) z[r] = 0.0f;
                    acc = Mfma<T>::mma(qa, kf[0], z);
                }
            } else {
                acc = Mfma<T>::mma(qa, kf[ks], acc);           // log2 P
            }
            dp = Mfma<T>::mma(ga, vf[ks], dp);                 // dP - delta
        }
        // consumed above; with registers to spare the next tile travels during the rest
        if (PREFETCH) load_btile(qtile + 1, ctile);
        if (R::RESID) {
#pragma unroll
            for (int ks = 0; ks < KSD; ++ks) {
                // (kres is zero in the lanes whose columns lie past the head dim: there this operand may hold
                // any finite values, and those lanes read the row's first chunk rather than being cleared per tile)
                const int ch = ks * 16 + g * 8 < D ? 2 * ks + g : 2 * ks;
                const v8 ql = *reinterpret_cast<const v8 *>(lds + OFF_QL + R::swz(qb + li, ch));
                acc = Mfma<T>::mma(ql, kres[ks], acc);
            }
        }
        float ds[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            acc[r] = fast_exp2(acc[r]);
            ds[r] = acc[r] * dp[r];
        }
        if (kill) {
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = 0.0f;
        }
        if (want_dm) {
#pragma unroll
            for (int r = 0; r < 16; ++r) dm += ds[r];
        }
        // all conversions before the gradient matmuls (measured 3 % faster than converting each
        // half right before its MFMAs)
        v8 pf2[2], dsf2[2];
#pragma unroll
        for (int ts = 0; ts < 2; ++ts)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                pf2[ts][i] = (T)acc[8 * ts + i];
                dsf2[ts][i] = (T)ds[8 * ts + i];
            }
#pragma unroll
        for (int ts = 0; ts < 2; ++ts) {
            const v8 pf = pf2[ts], dsf = dsf2[ts];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                // dO^T and Q^T fragments: row d = dt*32 + li, the 8 queries the P registers hold
                // Lanes whose column lies past the head dim (rows d >= D of the fragments: rows of dK^T and
                // dV^T that are never stored, and a row of the product depends on its own row of the A operand
                // only) read column 0 instead of being masked and cleared for every tile.
                const int col0 = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                const int col = (D % 32 == 0 || col0 < D) ? col0 : 0;
                v8 gta, qta;
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    const int row = qb + 16 * ts + 8 * h2 + 4 * g + ((lane & 15) >> 2);
                    const int o = R::swz(row, col >> 3) + (col & 7) * 2;
                    s16x4 rg = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4 __attribute__((address_space(3))) *)(lds + OFF_G + o));
                    s16x4 rq = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4 __attribute__((address_space(3))) *)(lds + OFF_QR + o));
                    v4 vg = __builtin_bit_cast(v4, rg), vq = __builtin_bit_cast(v4, rq);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        gta[4 * h2 + i] = vg[i];
                        qta[4 * h2 + i] = vq[i];
                    }
                }
                dv[dt] = Mfma<T>::mma(gta, pf, dv[dt]);
                dk[dt] = Mfma<T>::mma(qta, dsf, dk[dt]);
            }
        }
    };

    CTile ctile;
    if (PREFETCH) load_btile(0, ctile);
    stage(0);
    // K with the mask columns, V with ones against -delta
#pragma unroll
    for (int ks = 0; ks < KSD; ++ks) kres[ks] = zero8<T>();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int d0 = ks * 16 + g * 8;
        kf[ks] = zero8<T>();
        vf[ks] = zero8<T>();
        if (d0 < D) {
            if (!dead) kf[ks] = kraw[ks];
            if (ks < KSD) kres[ks] = kf[ks];   // against the residue columns of Q: data only
            vf[ks] = vraw[ks];
        } else if (d0 == AUGC) {
            kf[ks] = aug8<T>(mraw, one3);      // mask x ones, ones x -lse
            vf[ks] = aug8<T>(one3, zero3);     // ones x -delta
        }
    }
    for (int qtile = 0; qtile < NT; ++qtile) {
        if (qtile % TPS == 0 && qtile != 0) stage(qtile * 32);
        if (!PREFETCH) load_btile(qtile, ctile);
        if (active) compute(qtile, ctile);
        if (qtile < 8) EVO_TK(5 + qtile);
    }

    if (active) {
        if (want_dm) {
            dm += __shfl_xor(dm, 32);
            if (g == 0 && key < p.N) e.dmask_part[pr.row0 + key] = dm;
        }
        if (key < p.N) {
            T *dK = (T *)p.dk + pr.base + (int64_t)key * sn;
            T *dV = (T *)p.dv + pr.base + (int64_t)key * sn;
            const float kscale = p.scale;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                store_row_tile<T>(dK, dt * 32, D, dk[dt], kscale, g);
                store_row_tile<T>(dV, dt * 32, D, dv[dt], 1.0f, g);
            }
        }
    }
    EVO_TK(13);
}

// ------------------------------------------------------------------ launchers

template <typename T, int D, bool HAS_BIAS>
static int dq_ntw(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int NT = (p.N + 31) / 32;
    const unsigned grid = (unsigned)NT * (unsigned)(p.B * p.H) * (unsigned)e.n_chunks;
    const int ntw = (NT + 3) / 4;
    if (ntw <= 2) mfma_dq<T, D, HAS_BIAS, 2><<<grid, 256, 0, st>>>(p, e);
    else if (ntw <= 4) mfma_dq<T, D, HAS_BIAS, 4><<<grid, 256, 0, st>>>(p, e);
    else if (ntw <= 8) mfma_dq<T, D, HAS_BIAS, 8><<<grid, 256, 0, st>>>(p, e);
    else if (ntw <= 16) mfma_dq<T, D, HAS_BIAS, 16><<<grid, 256, 0, st>>>(p, e);
    else return EVO_EUNSUPPORTED;
    return hip_rc();
}

template <typename T, int D>
static int dq_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.bias_dtype == EVO_NONE ? dq_ntw<T, D, false>(p, e, st) : dq_ntw<T, D, true>(p, e, st);
}

template <typename T, int D, int BT, int NW, int ROWS>
static int dkdv_launch(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const unsigned grid = (unsigned)((p.N + NW * 32 - 1) / (NW * 32)) * (unsigned)(p.B * p.H * p.S);
    constexpr int lds = KvGeo<D>::lds_bytes(ROWS);   // at most 56 KB up to head dim 64, 100 KB at 128
    auto kern = mfma_dkdv<T, D, BT, NW, ROWS>;
    if constexpr (lds > 64 * 1024) {
        static PerDevice done{};
        if (const int rc = ensure_dynamic_lds((const void *)kern, lds, done, nullptr)) return rc;
    }
    kern<<<grid, NW * 64, lds, st>>>(p, e);
    return hip_rc();
}

template <typename T, int D, int NW>
static int dkdv_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    typedef KvGeo<D> R;
    const int bt = p.bias_dtype == EVO_NONE ? 0 : (e.bk16 && !e.bias_direct) ? 2 : 1;
    if (NW == 4 && p.N <= 128)
        return bt == 0 ? dkdv_launch<T, D, 0, NW, 128>(p, e, st)
             : bt == 2 ? dkdv_launch<T, D, 2, NW, 128>(p, e, st) : dkdv_launch<T, D, 1, NW, 128>(p, e, st);
    return bt == 0 ? dkdv_launch<T, D, 0, NW, R::BQS>(p, e, st)
         : bt == 2 ? dkdv_launch<T, D, 2, NW, R::BQS>(p, e, st) : dkdv_launch<T, D, 1, NW, R::BQS>(p, e, st);
}

// 8 waves (256 keys) per workgroup stage Q and dO once for twice the keys: measured faster
// wherever a problem has more than 128 keys (N = 256: 171 vs 191 us at S = 512, H = 8;
// N = 384, D = 32: 127 vs 149 us; N = 384, D = 8 within 3 %).
template <typename T, int D>
static int dkdv_waves(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    // EVO_FLAG_DEBUG_OTHER_WIDTH inverts the choice, for comparison
    // ... unless there are too few problems for that: below four workgroups per CU (256 CUs) the
    // narrower form's twice as many workgroups fill the chip better
    const int64_t wgs = (int64_t)((p.N + 255) / 256) * p.B * p.H * p.S;
    // ... and unless the last 256-key workgroup of a problem would be at most half full at a small head dim, where
    // staging Q and dO a second time is cheap (bf16, S = 1024, H = 8, N = 384: 444 vs 531 us at head dim 8, 535 vs
    // 571 us at 16; N = 320, head dim 8: 171 vs 222 us; at head dim 32 the two forms are level, 124 vs 123 us)
    const int rem = p.N % 256;
    const bool half_empty = D <= 16 && rem > 0 && rem <= 128;
    const bool wide = (p.N > 128 && wgs >= 1024 && !half_empty) != ((p.flags & EVO_FLAG_DEBUG_OTHER_WIDTH) != 0);
    return wide ? dkdv_bias<T, D, 8>(p, e, st) : dkdv_bias<T, D, 4>(p, e, st);
}

int EVO_CAT(launch_mfma_dq_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? dq_bias<bf16_t, EVO_D>(p, e, st) : dq_bias<f16_t, EVO_D>(p, e, st);
}

int EVO_CAT(launch_mfma_dkdv_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? dkdv_waves<bf16_t, EVO_D>(p, e, st) : dkdv_waves<f16_t, EVO_D>(p, e, st);
}

}  // namespace evo
