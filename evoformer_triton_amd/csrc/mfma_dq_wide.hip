// dQ (and delta) for problems whose dBias is not a sum over S rows: no pair bias, a bias that
// takes no gradient, or a single S row per (batch, head), where dBias is dS itself and is
// written as it is formed.  Compiled once per head dim (-DEVO_D=8|16|32|64).
//
// Replaces the reference's `_attn_bwd_preprocess` (evoformer.py:299-326) and `_attn_bwd_dq`
// (:329-476) for that case: P = exp(score - LSE) recomputed (:452), dS = P * (dP - delta)
// (:456), dS cast to the input dtype before the matmul (:459), dQ scaled after it (:462).
//
// The kernel that also sums dBias gives every wave a few (query tile, key tile) pairs to keep
// for a whole chunk of S rows, which spreads the keys of one query row over several waves: a
// partial dQ per wave, summed through LDS once per row.  Without dBias nothing ties a wave to
// a key tile, so this kernel is the mirror image of the dK/dV kernel: a wave owns 32 query
// rows of one problem (b, h, s) (Q pre-multiplied by scale*log2(e), dO, -LSE and -delta in
// registers) and walks over all keys, which the workgroup (NW waves = NW*32 queries) stages
// in LDS, row-major and as given, up to ROWS at a time: K with the mask columns, V.  Scores
// are transposed (S^T = K Q^T, dP^T = V dO^T: a lane owns one query and 16 keys), so that
// dS^T in accumulator layout is the B operand of dQ^T += K^T dS^T, whose A operand comes
// from the same K rows by transposing LDS reads.  dQ is complete inside the wave.
#include "bwd_common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

template <int D>
struct DqWideGeo {
    static constexpr int C = D / 8;                          // 16-byte chunks per row
    static constexpr int RPB = 16 / C > 0 ? 16 / C : 1;      // rows per 256 bytes
    static constexpr int ROWS = D <= 32 ? 256 : 128;         // keys staged per round
    // [K][V][mask columns of K]
    static constexpr int OFF_K = 0, OFF_V = ROWS * D * 2, OFF_AK = 2 * ROWS * D * 2;
    static constexpr int LDS_BYTES = OFF_AK + ROWS * 16;
    static __device__ __forceinline__ int swz(int r, int c) { return r * (D * 2) + ((c ^ ((r / RPB) % C)) << 4); }
};

typedef short s16x4w __attribute__((ext_vector_type(4)));

// BT: 0 no bias; 1 fp32 tiles (times log2 e) or, for very few S rows, the caller's rows; 2 the
// tiles of a bias in the dtype of q as given (half the bytes per tile; unpacked and multiplied by
// log2 e as they arrive)
template <typename T, int D, int BT, int NW, bool WRITE_DS>
__global__ void __launch_bounds__(NW * 64, D >= 128 ? 1 : NW == 8 ? (D <= 32 ? 4 : 2) : 3) mfma_dq_wide(EvoAttnParams p, Extra e) {
    constexpr bool HAS_BIAS = BT != 0, TILE16 = BT == 2;
    typedef Geo<D> G;
    typedef DqWideGeo<D> R;
    constexpr int KS = G::KS, KSD = G::KSD, DT = G::DT, AUGC = G::AUGC;
    constexpr int NTH = NW * 64, BQ = NW * 32, ROWS = R::ROWS, C = R::C, TPS = ROWS / 32;
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v4 v4;

    __shared__ __attribute__((aligned(1024))) unsigned char lds[R::LDS_BYTES];

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
    const T *Gd = (const T *)p.dout + pr.base;
    // (where delta is given, by the gate's pass, there may be no ungated O: the loads go to dO instead and their sum is dropped)
    const T *O = e.delta_given ? Gd : (const T *)p.o + pr.base;
    const int64_t sn = p.stride_n;
    const bool active = q0 < p.N;   // wave-uniform
    const int qrow = min(q0 + li, p.N - 1);
    const uint2 *m2row = e.m2 + ((int64_t)pr.b * p.S + pr.s) * npad;
    const bool dead = e.dead[pr.b * p.S + pr.s] != 0;
    const bool kill = dead && p.mask_kind == EVO_MASK_BOOL;
    const float cs = p.scale * kLog2e;
    const uint2 one3 = ones3<T>();
    const uint2 zero3 = {0u, 0u};

    // bias tile (query tile of this wave, key tile kt) in log2 units and accumulator order, or
    // this lane's row of the caller's tensor where no tiles were prepared
    const int bb = e.bias_batches > 1 ? pr.b : 0;
    const int qtc = min(q0 >> 5, NT - 1);
    const float *btile0 = e.bq + ((((int64_t)bb * p.H + pr.h) * NT + qtc) * NT) * 1024 + lane * 16;
    const float *ztile = e.bq + e.zero_tile + lane * 16;
    const bool bdirect = HAS_BIAS && e.bias_direct;
    const bool bf32 = p.bias_dtype == EVO_F32;
    const char *brow = (const char *)p.bias + ((int64_t)bb * p.bias_stride_b + (int64_t)pr.h * p.bias_stride_h +
                                               (int64_t)qrow * p.bias_stride_row) * (bf32 ? 4 : 2);
    const unsigned short *btile16 = !TILE16 ? nullptr
                                    : dead  ? e.bq16 + e.zero_tile + lane * 16
                                            : e.bq16 + ((((int64_t)bb * p.H + pr.h) * NT + qtc) * NT) * 1024 + lane * 16;
    auto load_btile = [&](int kt, f32x16 &dst) {
        if constexpr (TILE16) {
            Tile16 t;
            load_tile16(btile16 + (dead ? 0 : (int64_t)kt * 1024), t);
            unpack_tile16<T>(t, dead ? 0.0f : kLog2e, dst);
            return;
        }
        if (bdirect) {   // uniform
            const float mul = dead ? 0.0f : kLog2e;
            if (bf32) bias_tile_rows<T, true>(brow, kt * 32, p.N, g, mul, dst);
            else bias_tile_rows<T, false>(brow, kt * 32, p.N, g, mul, dst);
            return;
        }
        const float *src = dead ? ztile : btile0 + (int64_t)kt * 1024;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const f32x4 v = *reinterpret_cast<const f32x4 *>(src + 4 * rr);
            dst[4 * rr] = v[0]; dst[4 * rr + 1] = v[1]; dst[4 * rr + 2] = v[2]; dst[4 * rr + 3] = v[3];
        }
    };

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
    if (!e.delta_given && g == 0 && q0 + li < p.N) e.delta[pr.row0 + q0 + li] = dl;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        if (ks * 16 + g * 8 == AUGC) {
            qf[ks] = aug8<T>(one3, pack_split3<T>(-lse2));   // ones x mask, -lse x ones
            gf[ks] = aug8<T>(pack_split3<T>(-dl), zero3);    // -delta x ones
        }
    }
    const v8 vaug = aug8<T>(one3, zero3);                    // the V side of the -delta columns

    // S = 1: this lane's row of dBias[b][h] (reference: the atomic add of dS, evoformer.py:458,
    // with a single term)
    const int64_t dsrow = (((int64_t)pr.b * p.H + pr.h) * p.N + qrow) * p.N;
    const bool ds_vec = (p.N & 3) == 0 && ((uintptr_t)p.dbias & 15) == 0;
    const bool ds_f32 = p.dbias_dtype == EVO_F32;

    f32x16 dqacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) dqacc[dt][r] = 0.0f;

    // keys k0 .. k0 + ROWS - 1 into LDS: all loads first, then the writes (one round trip)
    auto stage = [&](int k0) {
        __syncthreads();
        constexpr int NIT = (ROWS * C + NTH - 1) / NTH;
        v8 kv[NIT], vv[NIT];
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int it = tid + i * NTH;
            const int row = min(it / C, ROWS - 1), ch = it % C, key = min(k0 + row, p.N - 1);
            kv[i] = ld8(K + (int64_t)key * sn + ch * 8);
            vv[i] = ld8(V + (int64_t)key * sn + ch * 8);
        }
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int it = tid + i * NTH;
            if (it < ROWS * C) {
                const int o = R::swz(it / C, it % C);
                *reinterpret_cast<v8 *>(lds + R::OFF_K + o) = kv[i];
                *reinterpret_cast<v8 *>(lds + R::OFF_V + o) = vv[i];
            }
        }
        // keys past the row's end carry the mask floor (prepared so): their probabilities vanish
        for (int row = tid; row < ROWS; row += NTH)
            *reinterpret_cast<v8 *>(lds + R::OFF_AK + row * 16) = aug8<T>(m2row[min(k0 + row, npad - 1)], one3);
        __syncthreads();
    };

    // this wave's 32 queries against key tile kt (staged at row kb of the buffer)
    auto compute = [&](int kt, int kb) {
        f32x16 acc, dp;
        if (HAS_BIAS) {
            load_btile(kt, acc);
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) dp[r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 16 + g * 8;
            v8 ka = zero8<T>(), va = zero8<T>();
            if (d0 < D) {
                const int o = R::swz(kb + li, 2 * ks + g);
                ka = *reinterpret_cast<const v8 *>(lds + R::OFF_K + o);
                va = *reinterpret_cast<const v8 *>(lds + R::OFF_V + o);
            } else if (d0 == AUGC || G::aug_step(ks)) {   // (qf, gf are zero in the step's upper half)
                ka = *reinterpret_cast<const v8 *>(lds + R::OFF_AK + (kb + li) * 16);
                va = vaug;
            }
            acc = Mfma<T>::mma(ka, qf[ks], acc);                                   // log2 P^T
            if (G::RESID && ks < KSD) acc = Mfma<T>::mma(ka, qlo[ks], acc);
            dp = Mfma<T>::mma(va, gf[ks], dp);                                     // dP^T - delta
        }
        float ds[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) ds[r] = fast_exp2(acc[r]) * dp[r];
        if (kill) {
#pragma unroll
            for (int r = 0; r < 16; ++r) ds[r] = 0.0f;
        }
        if (WRITE_DS && q0 + li < p.N) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int kg = kt * 32 + 8 * rr + 4 * g;   // registers 4rr .. 4rr+3 hold keys kg .. kg+3
                if (ds_vec && kg + 4 <= p.N) {
                    if (ds_f32) {
                        f32x4 v;
                        v[0] = ds[4 * rr]; v[1] = ds[4 * rr + 1]; v[2] = ds[4 * rr + 2]; v[3] = ds[4 * rr + 3];
                        *reinterpret_cast<f32x4 *>((float *)p.dbias + dsrow + kg) = v;
                    } else {
                        store4<T>((T *)p.dbias + dsrow + kg, ds[4 * rr], ds[4 * rr + 1], ds[4 * rr + 2], ds[4 * rr + 3]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (kg + i < p.N) {
                            if (ds_f32) ((float *)p.dbias)[dsrow + kg + i] = ds[4 * rr + i];
                            else ((T *)p.dbias)[dsrow + kg + i] = (T)ds[4 * rr + i];
                        }
                }
            }
        }
        v8 dsf2[2];
#pragma unroll
        for (int ts = 0; ts < 2; ++ts)
#pragma unroll
            for (int i = 0; i < 8; ++i) dsf2[ts][i] = (T)ds[8 * ts + i];
#pragma unroll
        for (int ts = 0; ts < 2; ++ts) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                // K^T fragment: row d = dt*32 + li, the 8 keys the dS registers hold
                // lanes whose column lies past the head dim (rows of the product that are never stored; a row of the
                // product depends on its own row of this operand only) read column 0 instead of being masked and cleared
                const int col0 = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                const int col = (D % 32 == 0 || col0 < D) ? col0 : 0;
                v8 kta;
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    const int row = kb + 16 * ts + 8 * h2 + 4 * g + ((lane & 15) >> 2);
                    const int o = R::swz(row, col >> 3) + (col & 7) * 2;
                    s16x4w rk = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4w __attribute__((address_space(3))) *)(lds + R::OFF_K + o));
                    v4 vk = __builtin_bit_cast(v4, rk);
#pragma unroll
                    for (int i = 0; i < 4; ++i) kta[4 * h2 + i] = vk[i];
                }
                dqacc[dt] = Mfma<T>::mma(kta, dsf2[ts], dqacc[dt]);
            }
        }
    };

    for (int k0 = 0; k0 < p.N; k0 += ROWS) {
        stage(k0);
        if (active) {
            const int nt = min(TPS, NT - k0 / 32);
#pragma unroll 1
            for (int j = 0; j < nt; ++j) compute(k0 / 32 + j, j * 32);
        }
    }

    if (active && q0 + li < p.N) {
        T *dQ = (T *)p.dq + pr.base + (int64_t)(q0 + li) * sn;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) store_row_tile<T>(dQ, dt * 32, D, dqacc[dt], p.scale, g);
    }
}

// ------------------------------------------------------------------ launcher

// Four waves (128 queries) per workgroup measured faster than eight at every size tried (N = 128
// .. 2048, all head dims: 114 vs 120 us at N = 256, 298 vs 324 us at N = 1024); bit 0x100 of
// flags (not part of the public interface) selects eight, for comparison.
template <typename T, int D, int BT, bool WRITE_DS>
static int dqw_waves(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int nw = (p.flags & EVO_FLAG_DEBUG_OTHER_WIDTH) ? 8 : 4;
    const unsigned grid = (unsigned)((p.N + nw * 32 - 1) / (nw * 32)) * (unsigned)(p.B * p.H * p.S);
    if (nw == 8) mfma_dq_wide<T, D, BT, 8, WRITE_DS><<<grid, 512, 0, st>>>(p, e);
    else mfma_dq_wide<T, D, BT, 4, WRITE_DS><<<grid, 256, 0, st>>>(p, e);
    return hip_rc();
}

template <typename T, int D>
static int dqw_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    if (p.bias_dtype == EVO_NONE) return dqw_waves<T, D, 0, false>(p, e, st);
    const bool t16 = e.bq16 && !e.bias_direct;
    if (!p.dbias) return t16 ? dqw_waves<T, D, 2, false>(p, e, st) : dqw_waves<T, D, 1, false>(p, e, st);
    if (p.S != 1) return EVO_EUNSUPPORTED;   // a sum over S rows is the other kernels' business
    return t16 ? dqw_waves<T, D, 2, true>(p, e, st) : dqw_waves<T, D, 1, true>(p, e, st);
}

int EVO_CAT(launch_mfma_dqw_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? dqw_bias<bf16_t, EVO_D>(p, e, st) : dqw_bias<f16_t, EVO_D>(p, e, st);
}

}  // namespace evo
