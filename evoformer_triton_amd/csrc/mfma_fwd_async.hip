// Persistent, asynchronously staged forward for gfx950.  Compiled once per head dim.
//
// Same arithmetic as mfma_fwd.hip (the reference's `_attn_fwd`, evoformer.py:23-297); what
// differs is how operands reach the matrix core.  Measured on MI355X, a workgroup that
// loads its 48 KB of K, V and Q in one burst waits 3 to 13 us for them under load, longer
// than it then computes.  Here one workgroup per CU stays resident and walks over its
// share of the (problem, 256-query block) items:
//   * two producer waves do nothing but issue `global_load_lds_dwordx4` for K, V, the
//     mask columns and Q of stages up to NB-1 ahead, straight into LDS ring buffers (no
//     registers, no vector ALU), and wait for the oldest stage in flight;
//   * eight consumer waves (32 query rows each) run the online softmax out of LDS.  Their
//     only global loads are the bias tiles (L2 resident), so the in-order completion of a
//     wave's vector loads never ties a consumer to an HBM round trip;
//   * one s_barrier per stage hands a filled buffer over and an emptied one back.
// K, V, Q rows sit in LDS row-major without padding; 16-byte chunks are XOR-swizzled by row
// so that the 16-byte operand reads and the transposing reads (`ds_read_b64_tr_b16`, which
// delivers V^T fragments from row-major V) are free of bank conflicts.  The swizzle is
// applied on the global side: lane i of a direct-to-LDS load always fills LDS slot i.
#include "common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

typedef short s16x4 __attribute__((ext_vector_type(4)));

template <int D>
struct AsyncGeo {
    static constexpr int C = D / 8;                          // 16-byte chunks per row
    static constexpr int RPB = 16 / C > 0 ? 16 / C : 1;      // rows per 256 bytes
    static constexpr int BKV = D <= 32 ? 256 : 128;          // keys per stage
    static constexpr int NB = D <= 32 ? 3 : 2;               // ring depth
    static constexpr int BQ = 256;                           // query rows per item (8 consumer waves)
    static constexpr int K_BYTES = BKV * D * 2;
    static constexpr int A_BYTES = BKV * 16;
    static constexpr int Q_BYTES = BQ * D * 2;
    static constexpr int OFF_V = K_BYTES;
    static constexpr int OFF_A = 2 * K_BYTES;
    static constexpr int OFF_Q = 2 * K_BYTES + A_BYTES;
    static constexpr int BUF_BYTES = 2 * K_BYTES + A_BYTES + Q_BYTES;
    static constexpr int LDS_BYTES = NB * BUF_BYTES;
    // direct-to-LDS instructions (1 KB each) per stage: K, V, mask columns, and Q on the
    // first stage of an item
    static constexpr int I_K = K_BYTES / 1024, I_A = A_BYTES / 1024, I_Q = Q_BYTES / 1024;
    static constexpr int I_KVA = 2 * I_K + I_A;
    // byte offset of chunk c of row r inside a swizzled row-major block
    static __device__ __forceinline__ int swz(int r, int c) { return r * (D * 2) + ((c ^ ((r / RPB) % C)) << 4); }
};

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding).
#define EVO_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x0F70)
// Bare workgroup barrier.  __syncthreads() would add a release fence, i.e. a wait for every
// outstanding vector load of the wave, which is exactly what the ring buffer must not do: a
// producer passes the barrier with younger stages still in flight, a consumer with its next
// bias tiles in flight.  What the hand-over needs is guaranteed otherwise: the producer has
// waited for the stage it hands over, and a consumer's LDS reads of a stage have all been
// consumed by MFMAs issued before it reaches the barrier.
#define EVO_BARRIER() asm volatile("s_barrier" ::: "memory")
#ifdef EVO_TRACE
#define EVO_T(slot)                                                                              \
    do {                                                                                         \
        if (e.trace && (threadIdx.x & 63) == 0 && (slot) < 16)                                   \
            e.trace[((int64_t)blockIdx.x * 10 + (threadIdx.x >> 6)) * 16 + (slot)] = wall_clock64(); \
    } while (0)
#else
#define EVO_T(slot) do {} while (0)
#endif

template <typename T, int D, bool HAS_BIAS>
__global__ void __launch_bounds__(640) mfma_fwd_async(EvoAttnParams p, Extra e) {
    typedef AsyncGeo<D> G;
    constexpr int C = G::C, BKV = G::BKV, NB = G::NB, BQ = G::BQ;
    constexpr int SPS = BKV / 64;                  // 64-key steps per stage
    constexpr int KSD = (D + 15) / 16;             // data k-steps
    constexpr bool AUG_IN_PAD = D == 8;            // mask columns share k-step 0 with the data
    constexpr int KS = AUG_IN_PAD ? 1 : KSD + 1;
    constexpr int DT = (D + 31) / 32;
    constexpr bool RESID = D <= 16;
    constexpr float TAU = 8.0f;
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v4 v4;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32;
    const int np256 = (p.N + 255) / 256 * 256;
    const int nqb = (p.N + BQ - 1) / BQ;
    const int nst = (p.N + BKV - 1) / BKV;          // stages per item
    const unsigned n_items = (unsigned)(p.B * p.H * p.S) * nqb;
    const unsigned first = blockIdx.x, stride = gridDim.x;
    const unsigned my_items = first < n_items ? (n_items - first + stride - 1) / stride : 0;
    const int T_total = (int)my_items * nst;        // stages this workgroup walks through
    const int64_t sn = p.stride_n;

    if (wave >= 8) {
        // ------------------------------------------------------------ producers
        const int pw = wave - 8;   // 0 or 1: even / odd instructions of a stage
        auto issue = [&](int t) {
            const unsigned item = first + (unsigned)(t / nst) * stride;
            const int st = t % nst, kv0 = st * BKV;
            const unsigned pid = item / nqb;
            const int qb0 = (item % nqb) * BQ;
            const Prob pr = decode_problem(p, pid);
            const T *Kp = (const T *)p.k + pr.base, *Vp = (const T *)p.v + pr.base, *Qp = (const T *)p.q + pr.base;
            const uint4 *Mp = e.m2a + ((int64_t)pr.b * p.S + pr.s) * np256 + kv0;
            unsigned char *buf = lds + (t % NB) * G::BUF_BYTES;
            const int ninst = G::I_KVA + (st == 0 ? G::I_Q : 0);
            for (int n = pw; n < ninst; n += 2) {
                const void *src;
                unsigned char *dst;
                if (n < 2 * G::I_K) {
                    const bool isv = n >= G::I_K;
                    const int L = (isv ? n - G::I_K : n) * 64 + lane;   // linear chunk = LDS slot
                    const int r = L / C, cpos = L % C;
                    const int ch = cpos ^ ((r / G::RPB) % C);           // global chunk that belongs there
                    const int key = min(kv0 + r, p.N - 1);
                    src = (isv ? Vp : Kp) + (int64_t)key * sn + ch * 8;
                    dst = buf + (isv ? G::OFF_V : 0) + (isv ? n - G::I_K : n) * 1024;
                } else if (n < G::I_KVA) {
                    const int m = n - 2 * G::I_K;
                    src = Mp + m * 64 + lane;
                    dst = buf + G::OFF_A + m * 1024;
                } else {
                    const int m = n - G::I_KVA;
                    const int L = m * 64 + lane;
                    const int r = L / C, cpos = L % C;
                    const int ch = cpos ^ ((r / G::RPB) % C);
                    const int row = min(qb0 + r, p.N - 1);
                    src = Qp + (int64_t)row * sn + ch * 8;
                    dst = buf + G::OFF_Q + m * 1024;
                }
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                                 (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
            }
        };
        EVO_T(0);
        for (int t = 0; t < NB - 1; ++t)
            if (t < T_total) issue(t);
        EVO_T(1);
        // stage 0 must have landed; only younger stages may still be in flight.  Their
        // instruction count varies (Q only on first stages of an item), so the bound is the
        // smallest a stage can have per producer; allowing fewer outstanding loads than are
        // really younger only waits longer.
        if (NB == 3 && T_total > 1) { EVO_WAIT_VM(G::I_KVA / 2); } else { EVO_WAIT_VM(0); }
        EVO_T(2);
        EVO_BARRIER();
        for (int k = 0; k < T_total; ++k) {
            if (k + NB - 1 < T_total) issue(k + NB - 1);
            // stage k+1 must have landed before the next hand-over; stage k+2 may be in flight
            if (NB == 3 && k + 2 < T_total) { EVO_WAIT_VM(G::I_KVA / 2); } else { EVO_WAIT_VM(0); }
            EVO_T(3 + 2 * k);
            EVO_BARRIER();
            EVO_T(4 + 2 * k);
        }
        return;
    }

    // ---------------------------------------------------------------- consumers
    const float cscale = p.scale * kLog2e;
    EVO_T(0);
    EVO_BARRIER();  // hand-over 0
    EVO_T(1);
    // Per-item context; the next item's is formed one item ahead so that its dead flag and
    // its first two bias tiles are requested before the current item's output stores.
    struct Ctx {
        Prob pr;
        int q0;
        bool active, dead;
        const float *btile;
        int64_t bstep;
    };
    auto make_ctx = [&](unsigned it) {
        Ctx c;
        const unsigned item = first + it * stride;
        c.pr = decode_problem(p, item / nqb);
        c.q0 = (item % nqb) * BQ + wave * 32;
        c.active = c.q0 < p.N;
        c.dead = e.dead[c.pr.b * p.S + c.pr.s] != 0;
        const int bb = e.bias_batches > 1 ? c.pr.b : 0;
        const int qt = min(c.q0 >> 5, NT - 1);
        c.btile = c.dead ? e.bq + e.zero_tile + lane * 16
                         : e.bq + ((((int64_t)bb * p.H + c.pr.h) * NT + qt) * NT) * 1024 + lane * 16;
        c.bstep = c.dead ? 0 : 1024;
        return c;
    };
    auto load_btile = [&](const Ctx &c, int kt, f32x16 &dst) {
        if (HAS_BIAS) {
            const float *src = c.btile + (int64_t)min(kt, NT - 1) * c.bstep;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(src + 4 * rr);
                dst[4 * rr] = v[0]; dst[4 * rr + 1] = v[1]; dst[4 * rr + 2] = v[2]; dst[4 * rr + 3] = v[3];
            }
        }
    };
    const int total_steps = (p.N + 63) / 64;
    f32x16 c0, c1;
    Ctx nxt = make_ctx(0);
    if (my_items > 0) {
        load_btile(nxt, 0, c0);
        load_btile(nxt, 1, c1);
    }
    int t = 0;
    for (unsigned it = 0; it < my_items; ++it) {
        const Ctx cur = nxt;
        if (it + 1 < my_items) nxt = make_ctx(it + 1);
        const Prob pr = cur.pr;
        const int q0 = cur.q0;
        const bool active = cur.active, dead = cur.dead;

        float m = -INFINITY, l = 0.0f;
        f32x16 oacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;
        v8 qf[KSD], qlo[KSD];

        for (int st = 0; st < nst; ++st, ++t) {
            const unsigned char *buf = lds + (t % NB) * G::BUF_BYTES;
            if (st == 0) {
                // this lane's half of its query row, pre-multiplied by scale*log2(e)
                const float cq = dead ? 0.0f : cscale;
#pragma unroll
                for (int ks = 0; ks < KSD; ++ks) {
                    const int ch = 2 * ks + g;
                    qf[ks] = zero8<T>();
                    qlo[ks] = zero8<T>();
                    if (ch < C) {
                        v8 raw = *reinterpret_cast<const v8 *>(buf + G::OFF_Q + G::swz(wave * 32 + li, ch));
                        scaled_hilo8<T>(raw, cq, qf[ks], qlo[ks]);
                    }
                }
            }
            if (active) {
                const int nsteps_here = min(SPS, (p.N - st * BKV + 63) / 64);
                // ---- scores of one 64-key step: S^T = K Q^T (+ bias tiles as C, + mask columns)
                auto qk = [&](int s4, f32x16 &a0, f32x16 &a1) {
                    const int kb = s4 * 64;
                    const int step = st * SPS + s4;
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        v8 k0, k1, qb;
                        if (ks < KSD) {
                            const int ch = 2 * ks + g;
                            if (AUG_IN_PAD && g == 1) {
                                k0 = *reinterpret_cast<const v8 *>(buf + G::OFF_A + (kb + li) * 16);
                                k1 = *reinterpret_cast<const v8 *>(buf + G::OFF_A + (kb + 32 + li) * 16);
                                qb = zero8<T>();
                                qb[0] = qb[1] = qb[2] = (T)1.0f;
                            } else {
                                k0 = *reinterpret_cast<const v8 *>(buf + G::swz(kb + li, ch < C ? ch : 0));
                                k1 = *reinterpret_cast<const v8 *>(buf + G::swz(kb + 32 + li, ch < C ? ch : 0));
                                qb = qf[ks];
                            }
                        } else {  // the mask k-step: columns 0..2 of lane group 0
                            k0 = zero8<T>();
                            k1 = zero8<T>();
                            qb = zero8<T>();
                            if (g == 0) {
                                k0 = *reinterpret_cast<const v8 *>(buf + G::OFF_A + (kb + li) * 16);
                                k1 = *reinterpret_cast<const v8 *>(buf + G::OFF_A + (kb + 32 + li) * 16);
                                qb[0] = qb[1] = qb[2] = (T)1.0f;
                            }
                        }
                        if (ks == 0) {
                            if (HAS_BIAS) {
                                a0 = Mfma<T>::mma(k0, qb, c0);
                                a1 = Mfma<T>::mma(k1, qb, c1);
                            } else {
                                f32x16 z;
#pragma unroll
                                for (int r = 0; r < 16; ++r) z[r] = 0.0f;
                                a0 = Mfma<T>::mma(k0, qb, z);
                                a1 = Mfma<T>::mma(k1, qb, z);
                            }
                        } else {
                            a0 = Mfma<T>::mma(k0, qb, a0);
                            a1 = Mfma<T>::mma(k1, qb, a1);
                        }
                        if (RESID && ks < KSD) {
                            v8 ql = (AUG_IN_PAD && g == 1) ? zero8<T>() : qlo[ks];
                            a0 = Mfma<T>::mma(k0, ql, a0);
                            a1 = Mfma<T>::mma(k1, ql, a1);
                        }
                    }
                    // the bias registers are free again: request the tiles of the next step
                    // (or of the next item's first step)
                    if (step + 1 < total_steps) {
                        load_btile(cur, 2 * step + 2, c0);
                        load_btile(cur, 2 * step + 3, c1);
                    } else {
                        load_btile(nxt, 0, c0);
                        load_btile(nxt, 1, c1);
                    }
                };
                // ---- online softmax of one step and O^T += V^T P^T
                auto softmax_pv = [&](int s4, f32x16 &a0, f32x16 &a1) {
                    const int kb = s4 * 64;
                    float mloc = fmaxf(a0[0], a1[0]);
#pragma unroll
                    for (int r = 1; r < 16; ++r) mloc = fmaxf(mloc, fmaxf(a0[r], a1[r]));
                    {   // exchange between the two lane groups without touching LDS
                        const unsigned u = __float_as_uint(mloc);
                        auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                        mloc = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
                    }
                    // rescale only when the max grows by more than 2^TAU
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
                    // V^T fragments by transposing reads of row-major V
#pragma unroll
                    for (int ts = 0; ts < 4; ++ts) {
                        v8 pf;
#pragma unroll
                        for (int i = 0; i < 8; ++i) pf[i] = (T)((ts < 2 ? a0 : a1)[8 * (ts & 1) + i]);
#pragma unroll
                        for (int dt = 0; dt < DT; ++dt) {
                            const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                            v8 va = zero8<T>();
                            if (col < D) {
#pragma unroll
                                for (int h2 = 0; h2 < 2; ++h2) {
                                    const int row = kb + 16 * ts + 8 * h2 + 4 * g + ((lane & 15) >> 2);
                                    const unsigned char *ad = buf + G::OFF_V + G::swz(row, col >> 3) + (col & 7) * 2;
                                    s16x4 rd = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                        (s16x4 __attribute__((address_space(3))) *)ad);
                                    v4 rv = __builtin_bit_cast(v4, rd);
                                    va[4 * h2] = rv[0]; va[4 * h2 + 1] = rv[1]; va[4 * h2 + 2] = rv[2]; va[4 * h2 + 3] = rv[3];
                                }
                            }
                            oacc[dt] = Mfma<T>::mma(va, pf, oacc[dt]);
                        }
                    }
                };
                // Two score register sets: the matrix core works on the scores of step s+1
                // while the vector ALU does the softmax of step s.
                f32x16 sa0, sa1, sb0, sb1;
                qk(0, sa0, sa1);
                for (int s4 = 0; s4 < nsteps_here; s4 += 2) {
                    if (s4 + 1 < nsteps_here) qk(s4 + 1, sb0, sb1);
                    softmax_pv(s4, sa0, sa1);
                    if (s4 + 1 < nsteps_here) {
                        if (s4 + 2 < nsteps_here) qk(s4 + 2, sa0, sa1);
                        softmax_pv(s4 + 1, sb0, sb1);
                    }
                }
            }
            EVO_T(2 + 2 * t);
            EVO_BARRIER();  // this buffer goes back to the producers, the next one is ready
            EVO_T(3 + 2 * t);
        }

        if (active) {
            l += __shfl_xor(l, 32);
            const float inv = 1.0f / l;
            const int q = q0 + li;
            if (q < p.N) {
                T *O = (T *)p.o + pr.base + (int64_t)q * sn;
                if (g == 0) p.lse[pr.row0 + q] = (m + __log2f(l)) * kLn2;
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
}

template <typename T, int D, bool HAS_BIAS>
static int fwda_launch(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    typedef AsyncGeo<D> G;
    static int cus = 0;
    static bool attr_set = false;
    auto kern = mfma_fwd_async<T, D, HAS_BIAS>;
    if (!attr_set) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess) return EVO_EHIP - (int)hipGetLastError();
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        hipError_t err = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, G::LDS_BYTES);
        if (err != hipSuccess) return EVO_EHIP - (int)err;
        attr_set = true;
    }
    const unsigned n_items = (unsigned)(p.B * p.H * p.S) * (unsigned)((p.N + G::BQ - 1) / G::BQ);
    const unsigned grid = n_items < (unsigned)cus ? n_items : (unsigned)cus;
    kern<<<grid, 640, G::LDS_BYTES, st>>>(p, e);
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

template <typename T>
static int fwda_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.bias_dtype == EVO_NONE ? fwda_launch<T, EVO_D, false>(p, e, st) : fwda_launch<T, EVO_D, true>(p, e, st);
}

int EVO_CAT(launch_mfma_fwda_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? fwda_bias<bf16_t>(p, e, st) : fwda_bias<f16_t>(p, e, st);
}

}  // namespace evo
