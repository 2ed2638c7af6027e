// dBias partials for rows of more than 256 keys, as a kernel of its own.
// Compiled once per head dim (-DEVO_D=8|16|32|64).
//
// dBias[b][h] is the sum over the S rows of dS = P * (dP - delta) (reference: the atomic add of
// every dS tile, evoformer.py:458).  Summing it inside the dQ kernel ties every wave of that
// kernel to a few (query tile, key tile) pairs for a whole chunk of S rows, and with many key
// tiles per row that leaves a workgroup 32 queries for all the keys it stages (N = 768: dQ in
// 1.67 ms against 0.68 ms without the sum).  For such rows dQ comes from the kernel that knows
// nothing of dBias, and this kernel forms dS a second time: a workgroup of 4 waves owns a block
// of 128 queries x 128 keys (64 at head dim 64) of one (b, h) for a chunk of S rows, a wave 32
// queries x 4 (2) key tiles, whose running sums (64 registers) and bias tiles (32, as 16-bit
// pairs) stay resident.  Per S row the workgroup stages its keys (K with the mask columns, V)
// in LDS, the waves fetch their own query rows (Q, dO, LSE, delta, as written by the dQ kernel);
// both are requested one row ahead into registers, and the keys go to the other of two LDS
// buffers after the row's tiles: one barrier per row.  Per tile: two score MFMA chains, exp2, a
// multiply and 16 additions; no conversions, no gradient matmul.  One partial per chunk;
// `dbias_reduce` adds them in order.
#include "bwd_common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

template <int D>
struct DbGeo {
    static constexpr int C = D / 8;                          // 16-byte chunks per row
    static constexpr int RPB = 16 / C > 0 ? 16 / C : 1;      // rows per 256 bytes
    // keys, queries per workgroup; key tiles per wave (head dim 64: half the keys, its operands
    // take the registers of two tiles' sums and bias)
    static constexpr int TPW = D <= 32 ? 4 : 2, KB = TPW * 32, QB = 128;
    static constexpr int OFF_K = 0, OFF_V = KB * D * 2, OFF_AK = 2 * KB * D * 2;
    static constexpr int LDS_BYTES = OFF_AK + KB * 16;
    static __device__ __forceinline__ int swz(int r, int c) { return r * (D * 2) + ((c ^ ((r / RPB) % C)) << 4); }
};

// BF32: the bias is fp32 (its prepared tiles are fp32 in log2 units and stay resident as they are: twice the
// registers of the 16-bit pairs, nothing to unpack)
template <typename T, int D, bool BF32>
__global__ void __launch_bounds__(256, 2) mfma_dbias(EvoAttnParams p, Extra e) {
    typedef Geo<D> G;
    typedef DbGeo<D> R;
    constexpr int KS = G::KS, KSD = G::KSD, AUGC = G::AUGC;
    constexpr int NTH = 256, KB = R::KB, C = R::C, TPW = R::TPW;
    constexpr int NIT = (KB * C + NTH - 1) / NTH;            // 16-byte pieces of K (and of V) per thread and row
    typedef typename Mfma<T>::v8 v8;

    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * R::LDS_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: what depends on it branches and is addressed by the scalar unit
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32, npad = NT * 32;
    const int nqb = (p.N + R::QB - 1) / R::QB, nkb = (p.N + KB - 1) / KB;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const int kbi = lid % nkb;
    const int qbi = (lid / nkb) % nqb;
    const unsigned bh = (lid / (nkb * nqb)) % (unsigned)(p.B * p.H);
    const int c = lid / (nkb * nqb) / (unsigned)(p.B * p.H);
    const int b = bh / p.H, h = bh % p.H;
    const int q0 = qbi * R::QB + wave * 32, k0 = kbi * KB;
    const bool active = q0 < p.N;                 // wave-uniform
    const int qrow = min(q0 + li, p.N - 1);
    const int nt = min(TPW, NT - k0 / 32);        // key tiles of this block that exist (>= 1)
    const int64_t sn = p.stride_n;
    const float cs = p.scale * kLog2e;
    const uint2 one3 = ones3<T>();
    const uint2 zero3 = {0u, 0u};
    const v8 vaug = aug8<T>(one3, zero3);

    // bias tiles (this wave's query tile x the block's key tiles) in accumulator order, as the
    // 16-bit values of the caller's tensor, two to a register (the prepared 16-bit tiles).  Per
    // use they are unpacked and multiplied by log2(e) in fp32, the product the fp32 tiles hold.
    const int bb = e.bias_batches > 1 ? b : 0;
    const int qtc = min(q0 >> 5, NT - 1);
    unsigned bres[BF32 ? 1 : TPW][8];
    f32x16 bres32[BF32 ? TPW : 1];
    f32x16 dbacc[TPW];
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
        const int kt = min(k0 / 32 + j, NT - 1);
        const int64_t o = ((((int64_t)bb * p.H + h) * NT + qtc) * NT + kt) * 1024 + lane * 16;
        if constexpr (BF32) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(e.bq + o + 4 * rr);
                bres32[j][4 * rr] = v[0]; bres32[j][4 * rr + 1] = v[1]; bres32[j][4 * rr + 2] = v[2]; bres32[j][4 * rr + 3] = v[3];
            }
        } else {
            Tile16 t;
            load_tile16(e.bq16 + o, t);
#pragma unroll
            for (int i = 0; i < 8; ++i) bres[j][i] = t.w[i >> 2][i & 3];
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) dbacc[j][r] = 0.0f;
    }

    const int s_begin = c * e.chunk, s_end = min(p.S, s_begin + e.chunk);
    if (s_begin >= s_end) return;                 // uniform over the workgroup

    // one row ahead, in registers: the block's K, V and mask pieces of this thread, the wave's
    // own query rows
    v8 kv[NIT], vv[NIT], qraw[KSD], graw[KSD];
    uint2 mk = zero3;
    float lse_n = 0.0f, delta_n = 0.0f;
    auto fetch = [&](int s) {
        const Prob pr = decode_problem(p, bh * (unsigned)p.S + s);
        const T *Q = (const T *)p.q + pr.base, *K = (const T *)p.k + pr.base, *V = (const T *)p.v + pr.base;
        const T *Gd = (const T *)p.dout + pr.base;
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int it = tid + i * NTH;
            const int row = min(it / C, KB - 1), ch = it % C, key = min(k0 + row, p.N - 1);
            kv[i] = ld8(K + (int64_t)key * sn + ch * 8);
            vv[i] = ld8(V + (int64_t)key * sn + ch * 8);
        }
        if (tid < KB) mk = e.m2[((int64_t)b * p.S + s) * npad + min(k0 + tid, npad - 1)];
#pragma unroll
        for (int ks = 0; ks < KSD; ++ks) {
            const int d0 = min(ks * 16 + g * 8, D - 8);
            qraw[ks] = ld8(Q + (int64_t)qrow * sn + d0);
            graw[ks] = ld8(Gd + (int64_t)qrow * sn + d0);
        }
        lse_n = p.lse[pr.row0 + qrow];
        delta_n = e.delta[pr.row0 + qrow];
    };

    // keys of a row into the buffer of that row's parity
    auto stash = [&](int buf) {
        unsigned char *dst = lds + buf * R::LDS_BYTES;
#pragma unroll
        for (int i = 0; i < NIT; ++i) {
            const int it = tid + i * NTH;
            if (it < KB * C) {
                const int o = R::swz(it / C, it % C);
                *reinterpret_cast<v8 *>(dst + R::OFF_K + o) = kv[i];
                *reinterpret_cast<v8 *>(dst + R::OFF_V + o) = vv[i];
            }
        }
        if (tid < KB) *reinterpret_cast<v8 *>(dst + R::OFF_AK + tid * 16) = aug8<T>(mk, one3);
    };

    fetch(s_begin);
    stash(0);
    __syncthreads();
    for (int s = s_begin; s < s_end; ++s) {
        const bool dead = e.dead[b * p.S + s] != 0;
        const bool kill = dead && p.mask_kind == EVO_MASK_BOOL;
        const float bscale = dead ? 0.0f : kLog2e;   // a row with every key masked takes no bias
        const unsigned char *buf = lds + ((s - s_begin) & 1) * R::LDS_BYTES;
        // the wave's operands of this row: Q scaled (with its rounding residue for small head
        // dims), dO, ones against the mask columns, -LSE and -delta against ones
        v8 qf[KS], gf[KS], qlo[KSD];
#pragma unroll
        for (int ks = 0; ks < KSD; ++ks) qlo[ks] = zero8<T>();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 16 + g * 8;
            qf[ks] = zero8<T>();
            gf[ks] = zero8<T>();
            if (d0 < D) {
                gf[ks] = graw[ks < KSD ? ks : 0];
                if (!dead) scaled_hilo8<T>(qraw[ks < KSD ? ks : 0], cs, qf[ks], qlo[ks < KSD ? ks : 0]);
            } else if (d0 == AUGC) {
                qf[ks] = aug8<T>(one3, pack_split3<T>(-lse_n * kLog2e));
                gf[ks] = aug8<T>(pack_split3<T>(-delta_n), zero3);
            }
        }
        fetch(min(s + 1, s_end - 1));   // in flight during the row's tiles

        if (active) {
#pragma unroll
            for (int j = 0; j < TPW; ++j) {
                if (j < nt) {   // uniform
                    const int kb = j * 32;
                    f32x16 acc, dp;
                    if constexpr (BF32) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[r] = dead ? 0.0f : bres32[j][r];   // (uniform)
                    } else {
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            // unpack per use: expanded once and for all the tiles would take twice the
                            // registers (the empty statement "changes" the resident register in place, so
                            // that its expansion cannot be moved out of the loop over S, at no copy)
                            asm volatile("" : "+v"(bres[j][i]));
                            float lo, hi;
                            unpack2<T>(bres[j][i], lo, hi);
                            acc[2 * i] = lo * bscale;
                            acc[2 * i + 1] = hi * bscale;
                        }
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) dp[r] = 0.0f;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        const int d0 = ks * 16 + g * 8;
                        v8 ka = zero8<T>(), va = zero8<T>();
                        if (d0 < D) {
                            const int o = R::swz(kb + li, 2 * ks + g);
                            ka = *reinterpret_cast<const v8 *>(buf + R::OFF_K + o);
                            va = *reinterpret_cast<const v8 *>(buf + R::OFF_V + o);
                        } else if (d0 == AUGC || G::aug_step(ks)) {   // (qf, gf are zero in the step's upper half)
                            ka = *reinterpret_cast<const v8 *>(buf + R::OFF_AK + (kb + li) * 16);
                            va = vaug;
                        }
                        acc = Mfma<T>::mma(ka, qf[ks], acc);                                   // log2 P^T
                        if (G::RESID && ks < KSD) acc = Mfma<T>::mma(ka, qlo[ks], acc);
                        dp = Mfma<T>::mma(va, gf[ks], dp);                                     // dP^T - delta
                    }
                    if (!kill) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) dbacc[j][r] += fast_exp2(acc[r]) * dp[r];
                    }
                }
                // (the tiles are unrolled for static register indices; without a fence the
                // scheduler pulls the next tiles' LDS reads forward and the registers run out)
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the next row's keys into the other buffer (everybody left it at the barrier before this
        // row); one barrier per row
        stash(((s - s_begin) & 1) ^ 1);
        __syncthreads();
    }

    // the partial of this chunk: lane = query li, registers 4rr .. 4rr+3 = keys 8rr + 4g ..
    if (active && q0 + li < p.N) {
        float *part = e.dbias_part + ((((int64_t)c * p.B + b) * p.H + h) * p.N + (q0 + li)) * p.N;
        const bool v4ok = (p.N & 3) == 0;
#pragma unroll
        for (int j = 0; j < TPW; ++j) {
            const int kb = k0 + j * 32;
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

// Workgroups per chunk of S rows: one per (query block, key block, batch, head).
int64_t EVO_CAT(mfma_dbias_blocks_d, EVO_D)(const EvoAttnParams &p) {
    typedef DbGeo<EVO_D> R;
    return (int64_t)((p.N + R::QB - 1) / R::QB) * ((p.N + R::KB - 1) / R::KB) * p.B * p.H;
}

int EVO_CAT(launch_mfma_dbias_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const int64_t grid = EVO_CAT(mfma_dbias_blocks_d, EVO_D)(p) * e.n_chunks;
    if (grid <= 0 || grid > 0x7fffffff) return EVO_EOVERFLOW;
    const bool bf32 = p.bias_dtype == EVO_F32;
    if (p.dtype == EVO_BF16) {
        if (bf32) mfma_dbias<bf16_t, EVO_D, true><<<(unsigned)grid, 256, 0, st>>>(p, e);
        else mfma_dbias<bf16_t, EVO_D, false><<<(unsigned)grid, 256, 0, st>>>(p, e);
    } else {
        if (bf32) mfma_dbias<f16_t, EVO_D, true><<<(unsigned)grid, 256, 0, st>>>(p, e);
        else mfma_dbias<f16_t, EVO_D, false><<<(unsigned)grid, 256, 0, st>>>(p, e);
    }
    return hip_rc();
}

}  // namespace evo
