// dK, dV (and the dMask partials) over a chunk of S rows of one head, with the head's pair
// bias resident in registers.  Compiled once per head dim (-DEVO_D=8|16|32|64); built for
// head dim 32 and 129..256 residues, the shape class of MSA row attention.
//
// Same arithmetic as `mfma_dkdv` in mfma_bwd.hip (the reference's `_attn_bwd_dk_dv`,
// evoformer.py:479-630): a wave owns 32 keys and walks over the query tiles of a row,
// S = Q K^T in accumulator layout gives P and dS as B operands of dV^T += dO^T P and
// dK^T += Q^T dS.  What differs is where the operands come from.  There, one workgroup per
// (b, h, s) problem streams the bias as fp32 tiles, 4 N^2 bytes per problem through the CU's
// 64-byte-per-clock load path (a fifth of that kernel's time at N = 256), and starts every
// problem with loads that only the other workgroup of the CU hides.  Here
//   * a workgroup of 8 waves (one per CU) keeps one head for a chunk of S rows; the bias
//     columns of a wave's 32 keys stay in 64 registers as 16-bit values in accumulator
//     order, read once per chunk from a transposed copy that the prep kernel writes; a
//     conversion and one fp32 multiplication per entry make them the C operand of the score
//     MFMA, in log2 units;
//   * Q, dO, LSE and delta of row s+1 are requested a few pieces per query tile while row s
//     is computed out of one LDS buffer, and written (Q also scaled, LSE and delta as
//     operand columns) to the other; the wave's K and V rows of row s+1 travel in registers;
//   * one barrier per row.
#include "bwd_common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <int D>
struct KvRingGeo {
    static constexpr int C = D / 8;                          // 16-byte chunks per row
    static constexpr int RPB = 16 / C > 0 ? 16 / C : 1;      // rows per 256 bytes
    static constexpr int NQ = 256;                           // query rows per stage (the longest row)
    static constexpr int Q_BYTES = NQ * D * 2;
    static constexpr int OFF_QS = 0;                         // Q * scale * log2(e)
    static constexpr int OFF_QR = Q_BYTES;                   // Q as given
    static constexpr int OFF_G = 2 * Q_BYTES;                // dO
    static constexpr int OFF_AQ = 3 * Q_BYTES;               // (1, 1, 1, -LSE hi, mid, lo, 0, 0) per query
    static constexpr int OFF_AG = OFF_AQ + NQ * 16;          // (-delta hi, mid, lo, 0, ...) per query
    static constexpr int BUF_BYTES = OFF_AG + NQ * 16;
    static constexpr int LDS_BYTES = 2 * BUF_BYTES;
    // 1 KB pieces (64 lanes x 16 bytes): Q, dO, then one piece of 256 LSE values and one of delta
    static constexpr int I_Q = Q_BYTES / 1024;
    static constexpr int I_ALL = 2 * I_Q + 2;
    static __device__ __forceinline__ int swz(int r, int c) { return r * (D * 2) + ((c ^ ((r / RPB) % C)) << 4); }
};

__device__ __forceinline__ void lds_barrier_kv() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <typename T, int D, bool HAS_BIAS>
__global__ void __launch_bounds__(512) mfma_dkdv_ring(EvoAttnParams p, Extra e) {
    typedef Geo<D> G;
    typedef KvRingGeo<D> R;
    static_assert(!G::RESID && D >= 16, "built for head dims whose scaled Q is rounded once");
    constexpr int KS = G::KS, KSD = G::KSD, DT = G::DT, AUGC = G::AUGC, C = R::C;
    constexpr int IPW = (R::I_ALL + 7) / 8;   // most pieces one wave moves per stage
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v4 v4;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32, npad = NT * 32;
    // Where the heads lie inside a token (the per-head layout) a cache line holds rows of several heads: the heads
    // of a chunk of S rows then run on one XCD, behind one L2 (consecutive workgroup ids go round the XCDs).
    const unsigned wid = p.stride_h < p.stride_n ? xcd_remap(blockIdx.x, gridDim.x) : blockIdx.x;
    const unsigned bh = wid % (unsigned)(p.B * p.H);
    const int c = wid / (unsigned)(p.B * p.H);
    const int b = bh / p.H, h = bh % p.H;
    const int key0 = wave * 32;
    const bool active = key0 < p.N;           // wave-uniform
    const int key = key0 + li, keyc = min(key, p.N - 1);
    const int64_t sn = p.stride_n;
    const bool want_dm = e.dmask_part != nullptr && p.dmask != nullptr;
    const float cs = p.scale * kLog2e;
    const uint2 one3 = ones3<T>();
    const uint2 zero3 = {0u, 0u};

    // the dBias partials that the dQ kernel left are summed here, a slice per workgroup, while the first loads of the
    // kernel proper are still to come
    if (e.dbias_chunks > 0) sum_dbias_partials<512>(p, e, tid);

    const int s_begin = c * e.chunk, s_end = min(p.S, s_begin + e.chunk);
    const int nrows = s_end - s_begin;
    if (nrows <= 0) return;   // uniform over the workgroup
    // element offset of row 0 of problem (b, h, s_begin); S row s is (s - s_begin) * stride_s on
    const int64_t base0 = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h + (int64_t)s_begin * p.stride_s;

    // bias of this wave's keys in accumulator order, 16 bits per entry: lane = key li, entry
    // 4 k + i of query tile j is the query 32 j + 8 k + 4 g + i
    uint2 bres[HAS_BIAS ? 32 : 1];
    if (HAS_BIAS) {
        const int bb = e.bias_batches > 1 ? b : 0;
        const T *bcol = (const T *)e.bt + (((int64_t)bb * p.H + h) * p.N + keyc) * p.N;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            // groups past the row repeat its last one (those queries carry -LSE = floor)
            const int q0 = min((j >> 2) * 32 + 8 * (j & 3) + 4 * g, p.N - 4);
            bres[j] = *reinterpret_cast<const uint2 *>(bcol + q0);
        }
    }

    // ---- the stage of row s_begin + t lives in buffer t & 1: a list of 1 KB pieces (64 lanes x
    // 16 bytes); piece n belongs to wave n % 8.  Lane i of piece m of Q or dO fills LDS slot
    // 64 m + i of that block, which the swizzle assigns to some chunk of some row.
    u32x4 stg[IPW];
    struct Piece {
        const unsigned char *base;   // shared by the lanes, for the first row of the chunk
        int64_t row_step;            // bytes per S row
        unsigned lane_off;
        int dst;
    };
    Piece pc[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
        const int n = min(wave + 8 * i, R::I_ALL - 1);   // (a wave with fewer pieces repeats its last one)
        if (n >= 2 * R::I_Q) {
            const float *src = (n == 2 * R::I_Q ? p.lse : e.delta) + ((int64_t)bh * p.S + s_begin) * p.N;
            pc[i].base = reinterpret_cast<const unsigned char *>(src);
            pc[i].row_step = (int64_t)p.N * 4;
            pc[i].lane_off = (unsigned)min(4 * lane, p.N - 4) * 4u;
            pc[i].dst = n == 2 * R::I_Q ? R::OFF_AQ : R::OFF_AG;
        } else {
            const bool isg = n >= R::I_Q;
            const int m = isg ? n - R::I_Q : n;
            const T *base = isg ? (const T *)p.dout : (const T *)p.q;
            const int L = m * 64 + lane;
            const int r = L / C, cpos = L % C;
            const int ch = cpos ^ ((r / R::RPB) % C);
            const int row = min(r, p.N - 1);
            pc[i].base = reinterpret_cast<const unsigned char *>(base + base0);
            pc[i].row_step = p.stride_s * 2;
            pc[i].lane_off = (unsigned)(row * (int)sn + ch * 8) * 2u;
            pc[i].dst = (isg ? R::OFF_G : R::OFF_QS) + m * 1024;
        }
    }
    // Loads are unconditional (the row past the end repeats the last row) so that the staging
    // registers stay registers.
    auto fetch_piece = [&](int t, int i) {
        t = min(t, nrows - 1);
        stg[i] = *reinterpret_cast<const u32x4 *>(pc[i].base + t * pc[i].row_step + pc[i].lane_off);
    };
    auto stash_piece = [&](int t, int i) {
        const int n = wave + 8 * i;
        if (t >= nrows || n >= R::I_ALL) return;   // uniform
        unsigned char *buf = lds + (t & 1) * R::BUF_BYTES;
        if (n >= 2 * R::I_Q) {
            // four LSE (or delta) values of the queries 4 lane .. 4 lane + 3 become operand columns
            const bool is_lse = n == 2 * R::I_Q;
            const f32x4 v = __builtin_bit_cast(f32x4, stg[i]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int q = 4 * lane + j;
                if (q < R::NQ) {
                    v8 col;
                    if (is_lse) {
                        // rows past N get -LSE = floor: their probabilities vanish
                        const float nl = q < p.N ? -v[j] * kLog2e : kMaskFloor;
                        col = aug8<T>(one3, pack_split3<T>(nl));
                    } else {
                        col = aug8<T>(pack_split3<T>(q < p.N ? -v[j] : 0.0f), zero3);
                    }
                    *reinterpret_cast<v8 *>(buf + pc[i].dst + q * 16) = col;
                }
            }
        } else if (n >= R::I_Q) {
            *reinterpret_cast<u32x4 *>(buf + pc[i].dst + lane * 16) = stg[i];
        } else {
            // Q twice: as given (dK sums over it) and with scale*log2(e), rounded exactly as in
            // the forward (the scores)
            const v8 raw = __builtin_bit_cast(v8, stg[i]);
            *reinterpret_cast<v8 *>(buf + pc[i].dst + (R::OFF_QR - R::OFF_QS) + lane * 16) = raw;
            *reinterpret_cast<v8 *>(buf + pc[i].dst + lane * 16) = scaled8<T>(raw, cs);
        }
    };

    // this wave's K and V rows and mask columns, one S row ahead in registers
    v8 knext[KSD], vnext[KSD];
    uint2 mnext;
    const T *Kw = (const T *)p.k + base0 + (int64_t)keyc * sn;
    const T *Vw = (const T *)p.v + base0 + (int64_t)keyc * sn;
    const uint2 *Mw = e.m2 + ((int64_t)b * p.S + s_begin) * npad + min(key, npad - 1);
    auto fetch_kv = [&](int t) {
        t = min(t, nrows - 1);
#pragma unroll
        for (int ks = 0; ks < KSD; ++ks) {
            const int d0 = min(ks * 16 + g * 8, D - 8);
            knext[ks] = ld8(Kw + (int64_t)t * p.stride_s + d0);
            vnext[ks] = ld8(Vw + (int64_t)t * p.stride_s + d0);
        }
        mnext = Mw[(int64_t)t * npad];
    };

    // K with the mask columns, V with ones against -delta, of the row whose K, V rows have
    // arrived (no gradient through the scores of a row that a bool mask drops entirely:
    // dP - delta := 0; such a row's scores are its mask alone)
    v8 kf[KS], vf[KS];
    auto operands = [&](bool dead) {
        const bool kill = dead && p.mask_kind == EVO_MASK_BOOL;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = ks * 16 + g * 8;
            kf[ks] = zero8<T>();
            vf[ks] = zero8<T>();
            if (d0 < D) {
                if (!dead) kf[ks] = knext[ks];
                if (!kill) vf[ks] = vnext[ks];
            } else if (d0 == AUGC) {
                kf[ks] = aug8<T>(mnext, one3);                 // mask x ones, ones x -lse
                if (!kill) vf[ks] = aug8<T>(one3, zero3);      // ones x -delta
            }
        }
    };

#pragma unroll
    for (int i = 0; i < IPW; ++i) fetch_piece(0, i);
    fetch_kv(0);
#pragma unroll
    for (int i = 0; i < IPW; ++i) stash_piece(0, i);
    bool dead = uniform_load(e.dead + b * p.S + s_begin) != 0;
    operands(dead);

    for (int t = 0; t < nrows; ++t) {
        const int s = s_begin + t;
        const int64_t base = base0 + (int64_t)t * p.stride_s;
        const int64_t row0 = ((int64_t)bh * p.S + s) * p.N;
        const float bscale = dead ? 0.0f : kLog2e;   // a row with every key masked takes no bias
        lds_barrier_kv();   // the stage of this row is in LDS; everybody is done with the row before
        const unsigned char *buf = lds + (t & 1) * R::BUF_BYTES;

        f32x16 dk[DT], dv[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dk[dt][r] = dv[dt][r] = 0.0f;
        float dm = 0.0f;

#pragma unroll
        for (int qt = 0; qt < 8; ++qt) {
            // The next row's requests go out a few per query tile rather than all after the
            // barrier (eight waves asking at once queue up behind the CU's load path), and what
            // they returned is written to the other buffer (free since the barrier) before the
            // wave's K and V rows are requested into the registers that this frees.
            if (qt < 3) {
                constexpr int PPT = (IPW + 2) / 3;
#pragma unroll
                for (int i = qt * PPT; i < (qt + 1) * PPT && i < IPW; ++i) fetch_piece(t + 1, i);
            }
            if (qt == 5) {
#pragma unroll
                for (int i = 0; i < IPW; ++i) stash_piece(t + 1, i);
                fetch_kv(t + 1);
            }
            if (active && qt < NT) {   // uniform
                const int qb = qt * 32;
                f32x16 acc, dp;
                if (HAS_BIAS) {
                    // the bias tile in log2 units is where the score MFMAs start from
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        // (the pairs are unpacked per row: expanded once and for all they
                        // would take twice the registers)
                        // (the empty statement "changes" the resident registers in place: their
                        // expansion cannot be moved out of the loop over S, and no copy is made)
                        asm volatile("" : "+v"(bres[4 * qt + k].x), "+v"(bres[4 * qt + k].y));
                        float f0, f1, f2, f3;
                        unpack2<T>(bres[4 * qt + k].x, f0, f1);
                        unpack2<T>(bres[4 * qt + k].y, f2, f3);
                        acc[4 * k] = f0 * bscale; acc[4 * k + 1] = f1 * bscale;
                        acc[4 * k + 2] = f2 * bscale; acc[4 * k + 3] = f3 * bscale;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) dp[r] = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int d0 = ks * 16 + g * 8;
                    v8 qa = zero8<T>(), ga = zero8<T>();
                    if (d0 < D) {
                        const int o = R::swz(qb + li, 2 * ks + g);
                        qa = *reinterpret_cast<const v8 *>(buf + R::OFF_QS + o);
                        ga = *reinterpret_cast<const v8 *>(buf + R::OFF_G + o);
                    } else if (d0 == AUGC || G::aug_step(ks)) {   // (kf, vf are zero in the step's upper half)
                        qa = *reinterpret_cast<const v8 *>(buf + R::OFF_AQ + (qb + li) * 16);
                        ga = *reinterpret_cast<const v8 *>(buf + R::OFF_AG + (qb + li) * 16);
                    }
                    acc = Mfma<T>::mma(qa, kf[ks], acc);   // log2 P
                    dp = Mfma<T>::mma(ga, vf[ks], dp);     // dP - delta
                }
                float ds[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    acc[r] = fast_exp2(acc[r]);
                    ds[r] = acc[r] * dp[r];
                }
                if (want_dm) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) dm += ds[r];
                }
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
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        // dO^T and Q^T fragments: row d = dt*32 + li, the 8 queries the P registers hold
                        // lanes whose column lies past the head dim (rows of the product that are never stored; a row of the
                        // product depends on its own row of this operand only) read column 0 instead of being masked and cleared
                        const int col0 = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                        const int col = (D % 32 == 0 || col0 < D) ? col0 : 0;
                        v8 gta, qta;
#pragma unroll
                        for (int h2 = 0; h2 < 2; ++h2) {
                            const int row = qb + 16 * ts + 8 * h2 + 4 * g + ((lane & 15) >> 2);
                            const int o = R::swz(row, col >> 3) + (col & 7) * 2;
                            s16x4 rg = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                (s16x4 __attribute__((address_space(3))) *)(buf + R::OFF_G + o));
                            s16x4 rq = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                (s16x4 __attribute__((address_space(3))) *)(buf + R::OFF_QR + o));
                            v4 vg = __builtin_bit_cast(v4, rg), vq = __builtin_bit_cast(v4, rq);
#pragma unroll
                            for (int i = 0; i < 4; ++i) {
                                gta[4 * h2 + i] = vg[i];
                                qta[4 * h2 + i] = vq[i];
                            }
                        }
                        dv[dt] = Mfma<T>::mma(gta, pf2[ts], dv[dt]);
                        dk[dt] = Mfma<T>::mma(qta, dsf2[ts], dk[dt]);
                    }
                }
            }
            // the tiles are unrolled (the resident bias is indexed statically); without a fence
            // the scheduler pulls the next tiles' LDS reads forward and the registers run out
            __builtin_amdgcn_sched_barrier(0);
        }
        // The next row's K and V operands are formed here, before the row's own stores: what
        // waits for loads must not have the stores in front of it (vector memory operations
        // complete in order), and the wait is counted within the iteration.
        dead = uniform_load(e.dead + b * p.S + min(s + 1, s_end - 1)) != 0;
        operands(dead);

        if (active) {
            if (want_dm) {
                dm += __shfl_xor(dm, 32);
                // (a buffer store: the row's address is scalar and the lane adds its key, formed here from the lane
                // number: an address or an offset per lane kept across the rows would be one or two registers spilled)
                const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(e.dmask_part + row0), 0, p.N * 4, 0x00020000);
                unsigned ln;
                asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
                if (g == 0 && key < p.N) __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(dm), rs, (int)((key0 + (ln & 31)) * 4), 0, 0);
            }
            if (key < p.N) {
                T *dK = (T *)p.dk + base + (int64_t)key * sn;
                T *dV = (T *)p.dv + base + (int64_t)key * sn;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    store_row_tile<T>(dK, dt * 32, D, dk[dt], p.scale, g);
                    store_row_tile<T>(dV, dt * 32, D, dv[dt], 1.0f, g);
                }
            }
        }
    }
}

// ------------------------------------------------------------------ launcher

template <typename T, int D, bool HAS_BIAS>
static int kvr_launch(const EvoAttnParams &p, const Extra &e0, hipStream_t st) {
    typedef KvRingGeo<D> R;
    static PerDevice done{};
    int cus = 256;
    auto kern = mfma_dkdv_ring<T, D, HAS_BIAS>;
    if (const int rc = ensure_dynamic_lds((const void *)kern, R::LDS_BYTES, done, &cus)) return rc;
    // one workgroup per CU: chunks of S rows such that (b, h, chunk) items about fill the chip
    // (these chunks are the kernel's own; the dBias partials keep theirs)
    Extra e = e0;
    const int bh = p.B * p.H;
    const int want = chunks_for_rounds(bh, p.S, cus, 0.0);
    e.chunk = (p.S + want - 1) / want;
    e.n_chunks = (p.S + e.chunk - 1) / e.chunk;
    kern<<<(unsigned)bh * (unsigned)e.n_chunks, 512, R::LDS_BYTES, st>>>(p, e);
    return hip_rc();
}

// Largest N this kernel takes for the head dim (0: not built for it; it takes N > 128 only).
int EVO_CAT(mfma_kvr_max_n_d, EVO_D)() { return EVO_D == 32 ? 256 : 0; }

int EVO_CAT(launch_mfma_kvr_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
#if EVO_D == 32
    const bool has_bias = p.bias_dtype != EVO_NONE;
    if (p.dtype == EVO_BF16)
        return has_bias ? kvr_launch<bf16_t, EVO_D, true>(p, e, st) : kvr_launch<bf16_t, EVO_D, false>(p, e, st);
    return has_bias ? kvr_launch<f16_t, EVO_D, true>(p, e, st) : kvr_launch<f16_t, EVO_D, false>(p, e, st);
#else
    (void)p; (void)e; (void)st;
    return EVO_EUNSUPPORTED;
#endif
}

}  // namespace evo
