// dQ, delta and dBias partials with the operands of each S row double-buffered in LDS.
// Compiled once per head dim (-DEVO_D=8|16|32|64).
//
// Same arithmetic as `mfma_dq` in mfma_bwd.hip (the reference's `_attn_bwd_preprocess` and
// `_attn_bwd_dq`, evoformer.py:299-476) and the same ownership: a workgroup keeps a slab of
// query rows of one head for a whole chunk of S rows, so that the running sum of dS for
// that slab (the dBias partial) and the slab's bias tiles stay in registers.  What differs
// is how the per-row operands arrive.  There, every S row starts with loads whose latency
// nothing hides (a few microseconds, several times the arithmetic of the row).  Here
//   * the workgroup has 8 waves and a slab of 64 query rows: wave w works on query tile
//     w / 4 and, of every block of keys, on the 32-key tiles (w % 4), (w % 4) + 4, ... (for
//     rows of more than one key block: 32 query rows, wave w on the key tiles w, w + 8, ...);
//   * K, V, the mask columns, and the slab's Q, dO and O rows of S row s+1 are requested
//     (16 bytes per lane and load, 6 loads per wave at D = 32) before row s is computed out
//     of one LDS buffer, and written to the other buffer when that arithmetic is done; rows
//     with more keys than one buffer holds go through it in blocks;
//   * K^T fragments for dQ^T += K^T dS^T come from row-major K by transposing LDS reads
//     (`ds_read_b64_tr_b16`), so no transposed copy is written.
// Staging through registers rather than with direct-to-LDS loads is deliberate: measured
// here, `global_load_lds_dwordx4` moves about 16 bytes per clock and CU and holds up the
// other waves' LDS reads while it does, a microsecond per S row; a 16-byte `ds_write` per
// lane does not.
#include <type_traits>

#include "bwd_common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif


namespace evo {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// QT: 32-row query tiles per workgroup (2, or 1 for rows of several key blocks: half the
// resident bias tiles and dBias accumulators per wave).
// KB: keys per stage (256; 128 for head dim 64, whose rows are long; 384 for rows of 257..384 keys at
// head dims 8 and 16, where a whole row fits one stage).
template <int D, int QT, int KB>
struct RingGeo {
    static constexpr int C = D / 8;                          // 16-byte chunks per row
    static constexpr int RPB = 16 / C > 0 ? 16 / C : 1;      // rows per 256 bytes
    static constexpr int BKV = KB;                           // keys per stage
    static constexpr int TPB = BKV / 32;                     // key tiles per stage
    static constexpr int KQ = 8 / QT;                        // waves per query tile, each with key tiles of its own
    static constexpr int TPW = TPB / KQ;                     // key tiles per stage and wave
    static constexpr int QR = 32 * QT;                       // query rows per workgroup
    static constexpr int DP = (D + 31) / 32 * 32;
    static constexpr int RP = DP;                            // pitch of a partial dQ row (floats); 16-byte pieces swizzled by row
    static constexpr int K_BYTES = BKV * D * 2;
    static constexpr int A_BYTES = BKV * 16;                 // the mask operand chunks as they lie in memory
    static constexpr int A_LDS = BKV * 8;                    // and in the stage: the three mask columns (hi, mid, lo, 0) alone
    static constexpr int Q_BYTES = QR * D * 2;
    static constexpr int OFF_V = K_BYTES;
    static constexpr int OFF_A = 2 * K_BYTES;
    static constexpr int OFF_Q = OFF_A + A_LDS;
    static constexpr int OFF_G = OFF_Q + Q_BYTES;
    static constexpr int OFF_O = OFF_G + Q_BYTES;
    static constexpr int OFF_L = OFF_O + Q_BYTES;                   // -log2-sum-exp of the QR query rows as (hi, mid, lo, 0)
    static constexpr int OFF_DL = OFF_L + QR * 8;                   // delta of the QR query rows (fp32), where it is given
    static constexpr int STAGE_BYTES = OFF_DL + QR * 4;
    static constexpr int RED_BYTES = 8 * 32 * RP * 4;
    static constexpr int STAGE_1K = (STAGE_BYTES + 1023) / 1024 * 1024;
    // The partial dQ tiles get LDS of their own where 160 KB allow it; otherwise they lie in the
    // buffer of the stage just consumed.  Where two such areas fit, the rows alternate between
    // them and a row needs no barrier between its tiles and the write of its partials.
    static constexpr bool OWN_RED = 2 * STAGE_1K + RED_BYTES <= 160 * 1024;
    static constexpr bool TWO_RED = 2 * STAGE_1K + 2 * RED_BYTES <= 160 * 1024;
    static constexpr int BUF_BYTES = OWN_RED ? STAGE_1K : ((STAGE_BYTES > RED_BYTES ? STAGE_BYTES : RED_BYTES) + 1023) / 1024 * 1024;
    static constexpr int LDS_BYTES = TWO_RED ? 2 * BUF_BYTES + 2 * RED_BYTES : OWN_RED ? 2 * BUF_BYTES + RED_BYTES : 2 * BUF_BYTES;
    // float offset of the 16-byte piece c4 of row r inside a partial dQ area (pieces XOR-swizzled by row: a
    // wave's 16-byte writes and the 16-byte reads of the sum both spread over all banks at a pitch of DP floats)
    static __device__ __forceinline__ int red_at(int r, int c4) { return r * RP + ((c4 ^ (r & 7)) << 2); }
    // 1 KB pieces (64 lanes x 16 bytes) per segment of a stage
    static constexpr int I_K = K_BYTES / 1024, I_A = A_BYTES / 1024, I_Q = Q_BYTES / 1024;
    static constexpr int I_KVA = 2 * I_K + I_A;
    static constexpr int I_ALL = I_KVA + 3 * I_Q;
    // byte offset of chunk c of row r inside a swizzled row-major block
    static __device__ __forceinline__ int swz(int r, int c) { return r * (D * 2) + ((c ^ ((r / RPB) % C)) << 4); }
};

// Workgroup barrier that orders LDS traffic only: the loads of the next stage and the stores
// of the last row stay in flight across it (__syncthreads() would wait for them).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#ifdef EVO_TRACE
// a cycle count per phase and wave for EVO_TRACE_ROWS rows of every workgroup's chunk, from its ninth row on
#define EVO_TRACE_ROWS 8
#define EVO_TR(slot)                                                                             \
    do {                                                                                         \
        if (e.trace && (threadIdx.x & 63) == 0 && s >= s_begin + 8 && s < s_begin + 8 + EVO_TRACE_ROWS)   \
            e.trace[(((int64_t)blockIdx.x * 8 + (threadIdx.x >> 6)) * EVO_TRACE_ROWS + (s - s_begin - 8)) * 16 + (slot)] = clock64(); \
    } while (0)
#else
#define EVO_TR(slot) do {} while (0)
#endif

// GATE: the gate's backward pass on the rows the kernel stages (the form of one stage of up to 256 keys at head
// dim 32): in place of dO and O the workgroup asks for the gradient of the gated output, the gate's logits and
// the gated output of its 64 query rows; the wave that holds a 1 KB piece of all three forms, as the gate's pass
// of its own does (generic.hip) and bit for bit like it, dO = dout * sigmoid(g) (to the stage, and to p.dout for
// the dK/dV kernel), dgate = dout * Og * (1 - sigmoid(g)) and delta = rowsum(dO * Og / sigmoid(g)) (to the
// stage and to e.delta).  Pieces 36..39 are then dout, 40..43 Q, 44..47 the logits, 52..55 Og (a piece and
// the two that follow it 8 and 16 numbers later belong to the same wave), 48..51 are not used.
// LH: the last key block of a row holds at most half a block of keys (rows of 257..384 keys in two blocks of 256): a wave
// has no tile in its upper half, and keeps neither bias nor dBias sums for one.
template <typename T, int D, bool HAS_BIAS, int NBLK, int QT, int KB, bool GATE = false, bool LH = false>
__global__ void __launch_bounds__(512) mfma_dq_ring(EvoAttnParams p, Extra e) {
    typedef Geo<D> G;
    typedef RingGeo<D, QT, KB> R;
    static_assert(R::TPW >= 1 && R::Q_BYTES % 1024 == 0, "query slab too small for this head dim");
    constexpr int KS = G::KS, KSD = G::KSD, DT = G::DT, AUGC = G::AUGC;
    constexpr int C = R::C, BKV = R::BKV, TPB = R::TPB, TPW = R::TPW, RP = R::RP, KQ = R::KQ, QR = R::QR;
    static_assert(!LH || (NBLK >= 2 && TPW % 2 == 0), "half a last block needs an even number of tiles per wave and stage");
    constexpr int NSLOT = NBLK * TPW - (LH ? TPW / 2 : 0);   // key tiles per wave over a whole row
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v4 v4;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar, so that what depends on it branches
    __builtin_assume(wave >= 0 && wave < 8);                     // (512 threads: lets piece numbers be bounded at compile time)
    const int li = lane & 31, g = lane >> 5;
    const int qi = wave / KQ, kq = wave % KQ;
    const int NT = (p.N + 31) / 32, NQP = (NT + QT - 1) / QT;
    const int np256 = (p.N + 255) / 256 * 256;
    const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
    const int qp = lid % NQP;
    const unsigned bh = (lid / NQP) % (unsigned)(p.B * p.H);
    const int c = lid / NQP / (unsigned)(p.B * p.H);
    const int b = bh / p.H, h = bh % p.H;
    const int qbase = qp * QR;
    const int q0 = qbase + qi * 32;
    const bool qact = q0 < p.N;             // wave-uniform; an odd tile count leaves one pair half empty
    const int qt = min(q0 >> 5, NT - 1);
    const int qrow = min(q0 + li, p.N - 1);
    const int64_t sn = p.stride_n;
    const bool want_dbias = e.dbias_part != nullptr && p.dbias != nullptr;
    const float cs = p.scale * kLog2e;

    f32x16 dbacc[NSLOT];
#pragma unroll
    for (int j = 0; j < NSLOT; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) dbacc[j][r] = 0.0f;

    // key tile of slot j of this wave
    auto slot_tile = [&](int j) { return (j / TPW) * TPB + (j % TPW) * KQ + kq; };

    f32x16 bres[HAS_BIAS ? NSLOT : 1];
    if (HAS_BIAS) {
        const int bb = e.bias_batches > 1 ? b : 0;
        // (tiles of a bias in the dtype of q are prepared as given, 16 bits per entry: log2 units here)
        const int64_t tile0 = ((((int64_t)bb * p.H + h) * NT + qt) * NT) * 1024 + lane * 16;
#pragma unroll
        for (int j = 0; j < NSLOT; ++j) {
            const int64_t o = tile0 + (int64_t)min(slot_tile(j), NT - 1) * 1024;
            if (e.bq16) {   // uniform
                Tile16 t;
                load_tile16(e.bq16 + o, t);
                unpack_tile16<T>(t, kLog2e, bres[j]);
            } else {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(e.bq + o + 4 * rr);
                    bres[j][4 * rr] = v[0]; bres[j][4 * rr + 1] = v[1]; bres[j][4 * rr + 2] = v[2]; bres[j][4 * rr + 3] = v[3];
                }
            }
        }
    }

    const int s_begin = c * e.chunk, s_end = min(p.S, s_begin + e.chunk);
    const int nrows = s_end - s_begin;
    const int T_total = nrows * NBLK;

    // ---- stage t = (row s_begin + t / NBLK, key block t % NBLK) lives in buffer t & 1.  It is a
    // list of 1 KB pieces (64 lanes x 16 bytes); piece n belongs to wave n % 8.  Lane i of
    // piece m of a row-major block fills LDS slot 64 m + i of that block, which the swizzle
    // assigns to some chunk of some row.
    static_assert(!GATE || (NBLK == 1 && QT == 2 && KB == 256 && D == 32), "the gate's pass is built into one form");
    constexpr int I_ALL = GATE ? R::I_KVA + 5 * R::I_Q : R::I_ALL;   // pieces of a stage with query rows
    constexpr int IPW = (I_ALL + 7) / 8;   // most pieces one wave moves per stage
    struct Staged {
        u32x4 v[IPW];
        float lse;
        float dl;   // delta, where it is given
    };
    // element offset of row 0 of problem (b, h, s_begin); S row s is (s - s_begin) * stride_s on
    const int64_t base0 = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h + (int64_t)s_begin * p.stride_s;
    // Where piece n of key block blk comes from and goes to: a base that every lane shares for
    // the first S row of the chunk, its advance per S row (both in bytes), this lane's offset
    // from it, and the LDS offset inside the stage.
    struct Piece {
        const unsigned char *base;
        int64_t row_step;
        unsigned lane_off;
        int dst;
    };
    auto describe = [&](int n, int blk) __attribute__((always_inline)) {
        Piece d;
        if (n >= 2 * R::I_K && n < R::I_KVA) {
            const int m = n - 2 * R::I_K;
            d.base = reinterpret_cast<const unsigned char *>(e.m2a + ((int64_t)b * p.S + s_begin) * np256 + blk * BKV + m * 64);
            d.row_step = (int64_t)np256 * 16;
            d.lane_off = lane * 16u;
            d.dst = R::OFF_A + m * 512;
        } else {
            const T *base;
            int m, row0, off;
            if (n < R::I_K) { base = (const T *)p.k; m = n; row0 = blk * BKV; off = 0; }
            else if (n < 2 * R::I_K) { base = (const T *)p.v; m = n - R::I_K; row0 = blk * BKV; off = R::OFF_V; }
            else if (GATE) {
                const int kind = (n - R::I_KVA) / R::I_Q;   // dout, Q, logits, (unused: Q once more), Og
                m = (n - R::I_KVA) % R::I_Q; row0 = qbase; off = R::OFF_Q;
                if (kind == 0) { base = (const T *)e.gate_dout; off = R::OFF_G; }
                else if (kind == 2) base = (const T *)e.gate_logits;
                else if (kind == 4) base = (const T *)e.gate_og;
                else base = (const T *)p.q;
            }
            else if (n < R::I_KVA + R::I_Q) { base = (const T *)p.q; m = n - R::I_KVA; row0 = qbase; off = R::OFF_Q; }
            else if (n < R::I_KVA + 2 * R::I_Q) { base = (const T *)p.dout; m = n - R::I_KVA - R::I_Q; row0 = qbase; off = R::OFF_G; }
            else {   // (where delta is given there may be no ungated O: the piece is dO once more, and is not used)
                base = e.delta_given ? (const T *)p.dout : (const T *)p.o; m = n - R::I_KVA - 2 * R::I_Q; row0 = qbase; off = R::OFF_O;
            }
            const int L = m * 64 + lane;
            const int r = L / C, cpos = L % C;
            const int ch = cpos ^ ((r / R::RPB) % C);
            const int row = min(row0 + r, p.N - 1);
            d.base = reinterpret_cast<const unsigned char *>(base + base0);
            d.row_step = p.stride_s * 2;
            d.lane_off = (unsigned)(row * (int)sn + ch * 8) * 2u;
            d.dst = off + m * 1024;
        }
        return d;
    };
    // The descriptors of a wave's pieces are formed once, for key block 0.  A K, V or mask piece of a later block
    // lies a fixed number of bytes further on, the same for every lane (K and V: as long as its rows exist; they
    // are buffer loads there, whose rows at or beyond N read as zero instead of being clamped to the last row).
    Piece fixed[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) fixed[i] = describe(min(wave + 8 * i, I_ALL - 1), 0);
    const int kv_valid = (int)(((int64_t)(p.N - 1) * sn + D) * 2);   // bytes from a problem's first K (V) row to the end of its last
    const int kv_blk = BKV * (int)sn * 2, a_blk = BKV * 16;           // bytes from one key block to the next: K and V rows, mask chunks
    // Loads are unconditional (a wave with fewer pieces repeats its last one, the stage past
    // the end repeats the last stage) so that the staging registers stay registers.
    // A piece's address is a pointer that all lanes share, advanced by the scalar unit from S row
    // to S row, plus a 32-bit lane offset that never changes (and, for a later key block of the
    // row, the block's distance): no 64-bit multiplication per piece and row.
    const unsigned char *fptr[IPW];
    const float *flse = p.lse + ((int64_t)bh * p.S + s_begin) * p.N;   // of the row the pointers stand at
    const unsigned flse_off = (unsigned)min(qbase + lane, p.N - 1);
#pragma unroll
    for (int i = 0; i < IPW; ++i) fptr[i] = fixed[i].base;
    // moves the pointers from stage t to stage t + 1 (they stay at the last stage): to the next S row where
    // stage t + 1 is a row's first
    auto fetch_advance = [&](int t) {
        if (t + 1 > T_total - 1 || (NBLK != 1 && (t + 1) % NBLK != 0)) return;
#pragma unroll
        for (int i = 0; i < IPW; ++i) fptr[i] += fixed[i].row_step;
        flse += p.N;
    };
    // pieces [i0, i1) of stage t; the last piece takes the log-sum-exp along
    auto fetch_part = [&](Staged &stg, int t, int i0, int i1) __attribute__((always_inline)) {
        t = min(t, T_total - 1);
        const int row = t / NBLK, blk = t % NBLK;
        const int ninst = blk == 0 ? I_ALL : R::I_KVA;
#pragma unroll
        for (int i = 0; i < IPW; ++i) {
            if (i < i0 || i >= i1) continue;
            if (NBLK == 1) {
                stg.v[i] = *reinterpret_cast<const u32x4 *>(fptr[i] + fixed[i].lane_off);
            } else {
                const int n = wave + 8 * i;   // uniform
                if (n < 2 * R::I_K) {
                    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)fptr[i], 0, kv_valid, 0x00020000);
                    stg.v[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)fixed[i].lane_off, blk * kv_blk, 0);
                } else if (n < R::I_KVA) {
                    stg.v[i] = *reinterpret_cast<const u32x4 *>(fptr[i] + blk * a_blk + fixed[i].lane_off);
                } else if (blk == 0) {   // (the pieces with query rows belong to a row's first stage)
                    stg.v[i] = *reinterpret_cast<const u32x4 *>(fptr[i] + fixed[i].lane_off);
                }
            }
        }
        // the log-sum-exp of the slab's rows travels the same way (one value per lane; every
        // wave asks, wave 0 stores): a load whose result is carried into the next row's
        // prologue in a register would make that prologue wait for everything requested here
        if (i1 >= IPW && (NBLK == 1 || blk == 0)) {
            const float *lsrc = flse;
            stg.lse = lsrc[flse_off];
            // (delta has the layout of the log-sum-exp: the same offset from its own base)
            if (!GATE && e.delta_given) stg.dl = (e.delta + (lsrc - p.lse))[flse_off];
        }
    };
    auto fetch = [&](Staged &stg, int t) { fetch_part(stg, t, 0, IPW); };
    constexpr int SPLIT = IPW / 2;   // pieces asked for at the top of a row; the rest after its prologue
    // What every wave of a query tile would otherwise redo in its prologue is done once, by
    // the wave that writes the piece: Q goes to LDS scaled by scale*log2(e) (where the scaled
    // Q is rounded once; with the rounding residue carried along it goes as given), zeroed
    // for a row with every key masked, and the log-sum-exp as its three operand columns.
    constexpr bool PRESCALE = !G::RESID;
    bool stage_dead = PRESCALE && uniform_load(e.dead + b * p.S + s_begin) != 0;
    auto stash_part = [&](const Staged &stg, int t, int i0, int i1, int par) __attribute__((always_inline)) {   // par: the buffer of stage t, t & 1
        const int blk = t % NBLK;
        if (t >= T_total) return;   // uniform (one branch for the stage, none per piece where every wave has all its pieces)
        const int ninst = blk == 0 ? I_ALL : R::I_KVA;
        unsigned char *buf = lds + par * R::BUF_BYTES;
        const float cq = stage_dead ? 0.0f : cs;   // (the flag of the row this stage belongs to)
#pragma unroll
        for (int i = 0; i < IPW; ++i) {
            if (i < i0 || i >= i1) continue;
            const int n = wave + 8 * i;
            if ((NBLK == 1 && 8 * i + 7 < I_ALL) || n < ninst) {
                const int dst = fixed[i].dst;
                const int qkind = GATE && n >= R::I_KVA ? (n - R::I_KVA) / R::I_Q : -1;   // (GATE: dout, Q, logits, unused, Og)
                if (n >= 2 * R::I_K && n < R::I_KVA) {   // of a mask chunk (hi, mid, lo, 1, 1, 1, 0, 0) the first 8 bytes
                    *reinterpret_cast<uint2 *>(buf + dst + lane * 8) = make_uint2(stg.v[i][0], stg.v[i][1]);
                } else if (GATE && qkind == 0) {
                    // the gate's pass on this lane's 8 elements of one query row (generic.hip: gate_bwd_kernel)
                    if constexpr (GATE) {
                        const v8 a = __builtin_bit_cast(v8, stg.v[i]), gl = __builtin_bit_cast(v8, stg.v[i + 1 < IPW ? i + 1 : i]),
                                 og = __builtin_bit_cast(v8, stg.v[i + 2 < IPW ? i + 2 : i]);
                        v8 r_o, r_g;
                        float dsum = 0.0f;
#pragma unroll
                        for (int j = 0; j < 8; ++j) {
                            const float den = 1.0f + fast_exp2(-(float)gl[j] * kLog2e);
                            const float sg = __builtin_amdgcn_rcpf(den);
                            const float gr = (float)a[j], ogf = (float)og[j];
                            r_o[j] = (T)(gr * sg);
                            r_g[j] = (T)(gr * ogf * (1.0f - sg));
                            dsum = fmaf((float)r_o[j], ogf * den, dsum);
                        }
                        // the C lanes of a row are neighbours (the swizzle permutes their chunks in pairs and pairs of pairs)
#pragma unroll
                        for (int w = 1; w < C; w <<= 1) dsum += __shfl_xor(dsum, w);
                        *reinterpret_cast<v8 *>(buf + dst + lane * 16) = r_o;
                        const int L = (n - R::I_KVA) % R::I_Q * 64 + lane;
                        const int r = L / C;
                        if (L % C == 0) *reinterpret_cast<float *>(buf + R::OFF_DL + r * 4) = dsum;
                        if (qbase + r < p.N) {
                            // (the piece's element offset inside the tensors laid out like q: the row's, plus the lane's)
                            const int64_t goff = base0 + (int64_t)t * p.stride_s;
                            unsigned char *o_row = reinterpret_cast<unsigned char *>((T *)p.dout + goff) + fixed[i].lane_off;
                            unsigned char *g_row = reinterpret_cast<unsigned char *>((T *)e.gate_dgate + goff) + fixed[i].lane_off;
                            *reinterpret_cast<v8 *>(o_row) = r_o;
                            *reinterpret_cast<v8 *>(g_row) = r_g;
                            if (L % C == 0) e.delta[((int64_t)bh * p.S + s_begin + t) * p.N + qbase + r] = dsum;
                        }
                    }
                } else if (GATE && qkind >= 2) {
                    // (logits, Og: used above; the unused piece)
                } else if (PRESCALE && (GATE ? qkind == 1 : n >= R::I_KVA && n < R::I_KVA + R::I_Q)) {
                    *reinterpret_cast<v8 *>(buf + dst + lane * 16) = scaled8<T>(__builtin_bit_cast(v8, stg.v[i]), cq);
                } else {
                    *reinterpret_cast<u32x4 *>(buf + dst + lane * 16) = stg.v[i];
                }
            }
        }
        if (i1 >= IPW && wave == 0 && blk == 0 && lane < QR) {
            *reinterpret_cast<uint2 *>(buf + R::OFF_L + lane * 8) = pack_split3<T>(-stg.lse * kLog2e);
            if (!GATE && e.delta_given) *reinterpret_cast<float *>(buf + R::OFF_DL + lane * 4) = stg.dl;
        }
    };
    auto stash = [&](const Staged &stg, int t, int par) { stash_part(stg, t, 0, IPW, par); };

    // The partial dQ^T tiles of a query tile (one per wave that works on it, fp32) summed, scaled and stored as a
    // row of dQ.  The older wave of every SIMD (waves 0..3), which the issue arbitration favours and which would
    // otherwise wait at the next barrier for the younger one, does the sums: thread i of those 256 takes the
    // 16-byte pieces i, i + 256, ... of the slab's QR x D results.  What does not depend on the row is formed once.
    constexpr int NSUM = QR * (D / 4), NIT = (NSUM + 255) / 256;
    constexpr int RPP = 256 / (D / 4);          // query rows that one pass of the 256 threads covers
    // Where a pass covers whole query tiles (head dims up to 32), a thread's pieces are its first one plus a
    // step that all lanes share, in LDS as in memory: one offset each is kept, not one per piece.
    constexpr bool AFFINE = RPP % 32 == 0;
    constexpr int NK = AFFINE ? 1 : NIT;
    int sum_lds[NK];          // float offset of the first wave's partial inside a partial dQ area
    unsigned sum_goff[NK];    // byte offset of the piece from the first query row of the problem in dQ
#pragma unroll
    for (int j = 0; j < NK; ++j) {
        const int it = (tid & 255) + 256 * j;
        const int q = min(it / (D / 4), QR - 1), d4 = (it % (D / 4)) * 4;
        sum_lds[j] = R::red_at((q >> 5) * KQ * 32 + (q & 31), d4 >> 2);
        sum_goff[j] = (unsigned)((qbase + q) * (int)sn + d4) * 2u;
    }
    const int sum_q0 = qbase + (tid & 255) / (D / 4);   // the query row of the thread's first piece
    // `row` points at the problem's first row in dQ (shared by the lanes)
    auto sum_store = [&](const float *red, unsigned char *row) {
        if (wave >= 4) return;
        f32x4 part[NIT][KQ];
#pragma unroll
        for (int j = 0; j < NIT; ++j) {
            const int o = AFFINE ? sum_lds[0] + j * (RPP / 32) * KQ * 32 * RP : sum_lds[j < NK ? j : 0];
#pragma unroll
            for (int w = 0; w < KQ; ++w) part[j][w] = *reinterpret_cast<const f32x4 *>(&red[o + w * 32 * RP]);
        }
#pragma unroll
        for (int j = 0; j < NIT; ++j) {
            f32x4 sum = part[j][0];
#pragma unroll
            for (int w = 1; w < KQ; ++w) sum += part[j][w];
            const bool ok = (tid & 255) + 256 * j < NSUM && sum_q0 + j * RPP < p.N;
            unsigned char *dst = AFFINE ? row + (int64_t)j * RPP * sn * 2 + sum_goff[0] : row + sum_goff[j < NK ? j : 0];
            if (ok) store4<T>(reinterpret_cast<T *>(dst), sum[0] * p.scale, sum[1] * p.scale, sum[2] * p.scale, sum[3] * p.scale);
        }
    };
    unsigned char *dq_row = reinterpret_cast<unsigned char *>((T *)p.dq + base0);   // of the row whose partials are summed next
    // The sum of a row's partials waits until the next row's first stage barrier has been
    // passed: nobody writes where the partials lie before another barrier has followed, which
    // with several key blocks per row is the next stage barrier and with one is a barrier of
    // its own (XBAR) between the row's tiles and the write of its partials.
    static_assert(NBLK == 1 || R::OWN_RED, "rows of several key blocks keep the partials out of the stage buffers");
    constexpr bool XBAR = NBLK == 1 && !R::TWO_RED;
    // With the partials out of the stage buffers, the buffer of the next stage is free from
    // the stage barrier on: every wave asks for half of its pieces at the top of the row and
    // writes them to LDS between its two tiles, while other waves compute; the other half it
    // asks for after the row's prologue and writes after the tiles.
    constexpr bool MID = NBLK == 1 && R::OWN_RED && TPW >= 2;
    // where the partials of the row that ended with stage `stage` lie; par: stage & 1 (one stage per row: the row's parity)
    auto red_of = [&](int stage, int par) {
        return (float *)(lds + (R::TWO_RED ? 2 * R::BUF_BYTES + (NBLK == 1 ? par : stage / NBLK & 1) * R::RED_BYTES
                                : R::OWN_RED ? 2 * R::BUF_BYTES : par * R::BUF_BYTES));
    };

    Staged sa;
    fetch(sa, 0);
    fetch_advance(0);
    stash(sa, 0, 0);

    const uint2 one3 = ones3<T>();
    const uint2 zero3 = {0u, 0u};
    int t = 0;
    // One S row.  With one stage per row the rows are unrolled in pairs, so that which of the two
    // buffers a row reads (PAR = 0, 1) is known at compile time and every LDS address is a register
    // that never changes plus an immediate offset; PAR = -1: the stage number decides.
    auto do_row = [&](const int s, auto par_c) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        Staged &cur = sa, &nxt = sa;
        const unsigned pid = bh * (unsigned)p.S + s;
        Prob pr;
        pr.b = b; pr.h = h; pr.s = s;
        pr.base = base0 + (int64_t)(s - s_begin) * p.stride_s;
        pr.row0 = (int64_t)pid * p.N;
        const bool dead = uniform_load(e.dead + b * p.S + s) != 0;
        const bool kill = dead && p.mask_kind == EVO_MASK_BOOL;
        // for the stage with query rows that is written during this row: the next row's
        stage_dead = PRESCALE && uniform_load(e.dead + b * p.S + min(s + 1, s_end - 1)) != 0;

        v8 qf[KS], gf[KS], qlo[KSD];
        f32x16 dqacc[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) dqacc[dt][r] = 0.0f;
        const unsigned char *buf = lds;

#pragma unroll
        for (int blk = 0; blk < NBLK; ++blk, ++t) {
            EVO_TR(0);
            lds_barrier();   // stage t is in LDS; stage t-1 and the last reduction are done with
            EVO_TR(1);
            // The CU's load path takes a stage's 48 requests (D = 32) at 16 clocks each: half of
            // them go out now and half after the row's prologue rather than all queue up behind
            // it (where the staging writes cannot be split, the waves take turns instead).  With
            // few requests per wave there is nothing to gain.
            const bool early = !(NBLK == 1 && IPW >= 4) || (wave & 1) == 0;
            if (MID) fetch_part(nxt, t + 1, 0, SPLIT);
            else if (early) fetch(nxt, t + 1);
            EVO_TR(2);
            const int par = PAR >= 0 ? PAR : (t & 1);
            buf = lds + par * R::BUF_BYTES;
            if (blk == 0 && s > s_begin) {
                sum_store(red_of(t - 1, par ^ 1), dq_row);
                dq_row += p.stride_s * 2;
            }
            EVO_TR(3);

            if (blk == 0) {
                // this lane's half of the query row: Q (scaled), dO, and delta = <dO, O>
                const uint2 nlse3 = *reinterpret_cast<const uint2 *>(buf + R::OFF_L + (qi * 32 + li) * 8);
                float dpart = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KSD; ++ks) qlo[ks] = zero8<T>();
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const int d0 = ks * 16 + g * 8;
                    qf[ks] = zero8<T>();
                    gf[ks] = zero8<T>();
                    if (d0 < D) {
                        const int o = R::swz(qi * 32 + li, 2 * ks + g);
                        const v8 qraw = *reinterpret_cast<const v8 *>(buf + R::OFF_Q + o);
                        gf[ks] = *reinterpret_cast<const v8 *>(buf + R::OFF_G + o);
                        if (PRESCALE) qf[ks] = qraw;   // scaled (and zeroed for a dead row) when it was staged
                        else if (!dead) scaled_hilo8<T>(qraw, cs, qf[ks], qlo[ks < KSD ? ks : 0]);
                        if constexpr (!GATE) {   // (with the gate's pass delta lies in the stage, and there is no O)
                            const v8 oraw = *reinterpret_cast<const v8 *>(buf + R::OFF_O + o);
                            dpart = dot8<T>(gf[ks], oraw, dpart);
                        }
                    }
                }
                float dl;
                {
                    const unsigned u = __float_as_uint(dpart);
                    auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                    dl = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
                }
                if (GATE || e.delta_given) dl = *reinterpret_cast<const float *>(buf + R::OFF_DL + (qi * 32 + li) * 4);   // uniform
                else if (kq == 0 && g == 0 && q0 + li < p.N) e.delta[pr.row0 + q0 + li] = dl;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks * 16 + g * 8 == AUGC) {
                        qf[ks] = aug8<T>(one3, nlse3);                   // ones x mask, -lse x ones
                        gf[ks] = aug8<T>(pack_split3<T>(-dl), zero3);    // -delta x ones
                    }
                }
            }

            EVO_TR(4);
            if (MID) fetch_part(nxt, t + 1, SPLIT, IPW);
            else if (!early) fetch(nxt, t + 1);
            fetch_advance(t + 1);
            EVO_TR(5);
            {
#pragma unroll
                for (int jj = 0; jj < TPW; ++jj) {
                    if (LH && blk == NBLK - 1 && jj >= TPW / 2) continue;   // (known at compile time: both loops are unrolled)
                    // The two waves of a SIMD (w and w + 4) take turns at the higher issue priority, tile by tile
                    // (S = 512, N = 256, H = 8, head dim 32: 2 us of 145 less).  Only where a wave has two tiles per
                    // stage: with one, the turn would leave the younger wave ahead throughout, and the older one, which
                    // also sums the partial dQ, then ends its row late (rows of 384 and 768 keys: 8 % slower).
                    if (NBLK == 1 && TPW == 2) {
                        if (((jj ^ (wave >> 2)) & 1) != 0) __builtin_amdgcn_s_setprio(1);
                        else __builtin_amdgcn_s_setprio(0);
                    }
                    const int tb = jj * KQ + kq;         // tile inside the stage
                    const int kt = blk * TPB + tb;
                    if (MID && jj == TPW - 1) {
                        EVO_TR(6);
                        stash_part(cur, t + 1, 0, SPLIT, par ^ 1);
                        EVO_TR(7);
                    }
                    // wave-uniform; no gradient goes through the scores of a row that a bool mask drops
                    // entirely: its tiles are skipped, dQ stays zero and dBias unchanged
                    if (qact && kt < NT && !kill) {
                        const int slot = blk * TPW + jj;
                        v8 ka[KS], va[KS];
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            const int d0 = ks * 16 + g * 8;
                            ka[ks] = zero8<T>();
                            va[ks] = zero8<T>();
                            if (d0 < D) {
                                const int o = R::swz(tb * 32 + li, 2 * ks + g);
                                ka[ks] = *reinterpret_cast<const v8 *>(buf + o);
                                va[ks] = *reinterpret_cast<const v8 *>(buf + R::OFF_V + o);
                            } else if (d0 == AUGC || (D >= 16 && ks == KS - 1)) {
                                // The extra columns.  From head dim 16 on they have a k-step of their own, whose
                                // upper half (lane group 1) is zero on the query side: there the key side may hold
                                // any finite values, so both lane groups read the same columns and no lane is
                                // cleared or masked per tile.
                                ka[ks] = aug8<T>(*reinterpret_cast<const uint2 *>(buf + R::OFF_A + (tb * 32 + li) * 8), one3);  // mask x ones, ones x -lse
                                va[ks] = aug8<T>(one3, zero3);                                                 // ones x -delta
                            }
                        }
                        f32x16 acc, dp, z;
#pragma unroll
                        for (int r = 0; r < 16; ++r) z[r] = 0.0f;
                        // the bias tile is the C operand of the first score MFMA (uniform branch)
                        if (HAS_BIAS && !dead) acc = Mfma<T>::mma(ka[0], qf[0], bres[slot]);
                        else acc = Mfma<T>::mma(ka[0], qf[0], z);
                        dp = Mfma<T>::mma(va[0], gf[0], z);
                        if (G::RESID) acc = Mfma<T>::mma(ka[0], qlo[0], acc);
#pragma unroll
                        for (int ks = 1; ks < KS; ++ks) {
                            acc = Mfma<T>::mma(ka[ks], qf[ks], acc);   // log2 P^T
                            if (G::RESID && ks < KSD) acc = Mfma<T>::mma(ka[ks], qlo[ks], acc);
                            dp = Mfma<T>::mma(va[ks], gf[ks], dp);     // dP^T - delta
                        }
                        float ds[16];
#pragma unroll
                        for (int r = 0; r < 16; ++r) ds[r] = fast_exp2(acc[r]) * dp[r];
                        if (want_dbias) {
#pragma unroll
                            for (int r = 0; r < 16; ++r) dbacc[slot][r] += ds[r];
                        }
#pragma unroll
                        for (int ts = 0; ts < 2; ++ts) {
                            v8 dsf;
#pragma unroll
                            for (int i = 0; i < 8; ++i) dsf[i] = (T)ds[8 * ts + i];
#pragma unroll
                            for (int dt = 0; dt < DT; ++dt) {
                                // K^T fragment: row d = dt*32 + li, the 8 keys the dS^T registers hold
                                // lanes whose column lies past the head dim (rows of the product that are never stored; a row of the
                                // product depends on its own row of this operand only) read column 0 instead of being masked and cleared
                                const int col0 = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                                const int col = (D % 32 == 0 || col0 < D) ? col0 : 0;
                                v8 kta;
#pragma unroll
                                for (int h2 = 0; h2 < 2; ++h2) {
                                    const int row = tb * 32 + 16 * ts + 8 * h2 + 4 * g + ((lane & 15) >> 2);
                                    const unsigned char *ad = buf + R::swz(row, col >> 3) + (col & 7) * 2;
                                    s16x4 rd = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                        (s16x4 __attribute__((address_space(3))) *)ad);
                                    v4 rv = __builtin_bit_cast(v4, rd);
                                    kta[4 * h2] = rv[0]; kta[4 * h2 + 1] = rv[1]; kta[4 * h2 + 2] = rv[2]; kta[4 * h2 + 3] = rv[3];
                                }
                                dqacc[dt] = Mfma<T>::mma(kta, dsf, dqacc[dt]);
                            }
                        }
                    }
                }
            }
            EVO_TR(8);
            // into the other buffer, free since the barrier above
            if (MID) stash_part(cur, t + 1, SPLIT, IPW, par ^ 1);
            else if (R::OWN_RED) stash(cur, t + 1, par ^ 1);
        }

        // Partial dQ^T of this wave: lane = query li, register r = dim dt*32 + crow(r, g).  The
        // waves of a query tile meet in LDS.
        EVO_TR(9);
        if (XBAR) lds_barrier();
        const int lpar = PAR >= 0 ? PAR : ((t - 1) & 1);   // of the row's last stage
        float *red = red_of(t - 1, lpar);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                f32x4 v;
                v[0] = dqacc[dt][4 * rr]; v[1] = dqacc[dt][4 * rr + 1];
                v[2] = dqacc[dt][4 * rr + 2]; v[3] = dqacc[dt][4 * rr + 3];
                *reinterpret_cast<f32x4 *>(&red[R::red_at(wave * 32 + li, dt * 8 + 2 * rr + g)]) = v;
            }
        // where the partials share the stage buffers, the other buffer held the last row's;
        // everyone has summed them by now
        if (!R::OWN_RED) stash(cur, t, lpar ^ 1);
        EVO_TR(10);
    };
    if (NBLK == 1) {
        for (int s = s_begin; s < s_end; s += 2) {
            do_row(s, std::integral_constant<int, 0>{});
            if (s + 1 < s_end) do_row(s + 1, std::integral_constant<int, 1>{});
        }
    } else {
        for (int s = s_begin; s < s_end; ++s) do_row(s, std::integral_constant<int, -1>{});
    }
    if (s_end > s_begin) {
        lds_barrier();
        sum_store(red_of(t - 1, (t - 1) & 1), dq_row);
    }

    if (want_dbias && qact && q0 + li < p.N) {
        float *part = e.dbias_part + ((((int64_t)c * p.B + b) * p.H + h) * p.N + (q0 + li)) * p.N;
        const bool v4ok = (p.N & 3) == 0;
#pragma unroll
        for (int j = 0; j < NSLOT; ++j) {
            const int kb = slot_tile(j) * 32;
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

// ------------------------------------------------------------------ launcher

template <typename T, int D, bool HAS_BIAS, int NBLK, int QT, int KB, bool GATE = false, bool LH = false>
static int dqr_launch(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    typedef RingGeo<D, QT, KB> R;
    static PerDevice done{};
    auto kern = mfma_dq_ring<T, D, HAS_BIAS, NBLK, QT, KB, GATE, LH>;
    if (const int rc = ensure_dynamic_lds((const void *)kern, R::LDS_BYTES, done, nullptr)) return rc;
    const int NT = (p.N + 31) / 32, NQP = (NT + QT - 1) / QT;
    const unsigned grid = (unsigned)NQP * (unsigned)(p.B * p.H) * (unsigned)e.n_chunks;
    kern<<<grid, 512, R::LDS_BYTES, st>>>(p, e);
    return hip_rc();
}

// The forms the kernel is built in.  Per key tile of a row a wave keeps 16 registers of bias
// and 16 of dBias sums (three tiles per wave fit, four spill and run slower than the
// one-workgroup-per-problem kernel):
//   head dims 8, 16, 32   N <= 256        1 block of 256 keys, 2 query tiles per workgroup (2 tiles per wave)
//   head dims 8, 16       N <= 384        1 block of 384 keys, 2 query tiles               (3 tiles per wave; one stage and two
//                                         barriers per row: at head dim 16, S = 512, H = 8, N = 384 260 us against 330 us
//                                         for three blocks of 128 keys, at head dim 8, S = 1024 457 against 467 us for two
//                                         blocks of 256; at head dim 32 its stage and tiles together spill 113 registers)
//   head dim 8            N <= 512        2 blocks of 256 keys, 2 query tiles               (4 tiles per wave; its working set is small)
//   head dim 32           N <= 384        2 blocks of 256 keys, the second at most half full, 2 query tiles (3 tiles per
//                                         wave, two stages and barriers per row: N = 384, D = 32, S = 384, H = 4 129 us
//                                         against 142 us for three blocks of 128 keys, the form before)
//                         N <= 512, 768   2, 3 blocks of 256 keys, 1 query tile             (2, 3 tiles per wave)
//   head dim 64           N <= 128        1 block of 128 keys, 2 query tiles                (1 tile per wave)
struct DqrForm {
    int nblk, qt, kb;   // nblk = 0: not built for such rows
};
template <int D>
constexpr DqrForm dqr_form(int n) {
    if (D == 64) return n <= 128 ? DqrForm{1, 2, 128} : DqrForm{0, 0, 0};
    if (n <= 256) return DqrForm{1, 2, 256};
    if (D == 8) return n <= 384 ? DqrForm{1, 2, 384} : n <= 512 ? DqrForm{2, 2, 256} : DqrForm{0, 0, 0};
    if (n <= 384) return D == 16 ? DqrForm{1, 2, 384} : DqrForm{2, 2, 256};
    if (n <= 512) return DqrForm{2, 1, 256};
    if (n <= 768) return DqrForm{3, 1, 256};
    return DqrForm{0, 0, 0};
}

template <typename T, int D, bool HAS_BIAS>
static int dqr_blocks(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const DqrForm f = dqr_form<D>(p.N);
    if constexpr (D == 64) {
        if (f.nblk == 1) return dqr_launch<T, D, HAS_BIAS, 1, 2, 128>(p, e, st);
    } else {
        if constexpr (D == 32) {
            static_assert(dqr_form<32>(256).nblk == 1 && dqr_form<32>(256).qt == 2 && dqr_form<32>(256).kb == 256, "the form with the gate's pass");
            if (e.gate_dout) return mfma_dqr_gate_ok(D, p.N) ? dqr_launch<T, D, HAS_BIAS, 1, 2, 256, true>(p, e, st) : EVO_EINVAL;
        } else if (e.gate_dout) {
            return EVO_EINVAL;   // (the caller asks for the gate's pass only where this kernel has it)
        }
        if (f.nblk == 1 && f.kb == 256) return dqr_launch<T, D, HAS_BIAS, 1, 2, 256>(p, e, st);
        if constexpr (D == 8) {
            if (f.nblk == 1 && f.kb == 384) return dqr_launch<T, D, HAS_BIAS, 1, 2, 384>(p, e, st);
            if (f.nblk == 2) return dqr_launch<T, D, HAS_BIAS, 2, 2, 256>(p, e, st);
        } else {
            if constexpr (D == 16) {
                if (f.nblk == 1 && f.kb == 384) return dqr_launch<T, D, HAS_BIAS, 1, 2, 384>(p, e, st);
            } else {
                if (f.nblk == 2 && f.qt == 2) return dqr_launch<T, D, HAS_BIAS, 2, 2, 256, false, true>(p, e, st);
            }
            if (f.nblk == 2) return dqr_launch<T, D, HAS_BIAS, 2, 1, 256>(p, e, st);
            if (f.nblk == 3) return dqr_launch<T, D, HAS_BIAS, 3, 1, 256>(p, e, st);
        }
    }
    return EVO_EUNSUPPORTED;
}

template <typename T, int D>
static int dqr_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.bias_dtype == EVO_NONE ? dqr_blocks<T, D, false>(p, e, st) : dqr_blocks<T, D, true>(p, e, st);
}

// Query rows one workgroup of the double-buffered dQ kernel takes at this N (64 or 32); 0
// where the kernel is not built for such rows.
int EVO_CAT(mfma_dqr_qrows_d, EVO_D)(int n) { return 32 * dqr_form<EVO_D>(n).qt; }

int EVO_CAT(launch_mfma_dqr_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    return p.dtype == EVO_BF16 ? dqr_bias<bf16_t, EVO_D>(p, e, st) : dqr_bias<f16_t, EVO_D>(p, e, st);
}

}  // namespace evo
