// Forward for rows of at most 256 keys: one workgroup walks over a chunk of S rows of one
// head with the head's bias resident in registers.  Compiled once per head dim.
//
// Same arithmetic as mfma_fwd.hip (the reference's `_attn_fwd`, evoformer.py:23-297).  That
// kernel is one workgroup per (b, h, s) problem: every problem starts with loads whose
// latency nothing hides, and every problem reads its N x N bias tiles again (fp32, from L2),
// which at N = 256, D = 32 is four times the bytes of Q, K, V and O together.  Here
//   * a workgroup has 8 waves = 256 query rows (all of them) and a fixed head; wave w keeps
//     the bias of (query tile w) x (all keys) for the whole chunk of S rows, as it sits in
//     memory: 16-bit values, 64 registers, read once per chunk straight from the caller's
//     tensor.  It enters the scores through the matrix core, S^T = I B^T with I the identity
//     (2 MFMAs per 32 x 32 tile, exact), and is brought to log2 units by one fp32
//     multiplication per score;
//   * K, V and the mask columns of row s+1 are requested (16 bytes per lane and load) before
//     row s is computed out of one LDS buffer and written into the other one afterwards; a
//     wave's own Q rows are prefetched straight into its registers;
//   * the running maximum is folded into the next step's score MFMA as three more 16-bit
//     columns (next to the mask's), so that the scores arrive relative to it and the common
//     step does no subtraction; row sums are taken from the converted pairs (`v_dot2c`),
//     i.e. of exactly the probabilities that multiply V;
//   * V^T fragments come from row-major V by transposing LDS reads (`ds_read_b64_tr_b16`);
//   * one workgroup barrier per S row.
// K and V rows sit in LDS row-major without padding; 16-byte chunks are XOR-swizzled by row
// so that the operand reads and the transposing reads are free of bank conflicts.
// Needs the bias in the inputs' dtype with 16-byte aligned rows (N % 8 == 0); other cases
// run mfma_fwd.hip.
#include "bwd_common.h"
#include "kernels.h"

#ifndef EVO_D
#error "compile with -DEVO_D=<head dim>"
#endif

namespace evo {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <int D>
struct FwdRingGeo {
    static constexpr int C = D / 8;                          // 16-byte chunks per row
    static constexpr int RPB = 16 / C > 0 ? 16 / C : 1;      // rows per 256 bytes
    static constexpr int BKV = 256;                          // keys per stage = most keys per row
    static constexpr int K_BYTES = BKV * D * 2;
    static constexpr int A_BYTES = BKV * 16;
    static constexpr int OFF_V = K_BYTES;
    static constexpr int OFF_A = 2 * K_BYTES;
    static constexpr int BUF_BYTES = 2 * K_BYTES + A_BYTES;
    static constexpr int LDS_BYTES = 2 * BUF_BYTES;
    // 1 KB pieces (64 lanes x 16 bytes) per segment of a stage
    static constexpr int I_K = K_BYTES / 1024, I_A = A_BYTES / 1024;
    static constexpr int I_ALL = 2 * I_K + I_A;
    static __device__ __forceinline__ int swz(int r, int c) { return r * (D * 2) + ((c ^ ((r / RPB) % C)) << 4); }
};

// The gated form's copy of the gate logits in LDS: per wave its 32 query rows of D 16-bit values, in pieces of
// 64 lanes x 16 bytes (at head dim 8 half a piece holds them).
template <int D> constexpr int kGatePieces = D >= 16 ? D / 16 : 1;
template <int D> constexpr int kGateWaveBytes = kGatePieces<D> * 1024;
template <int D> constexpr int kGateBytes = 8 * kGateWaveBytes<D>;

// Workgroup barrier that orders LDS traffic only: the loads of the next row and the stores
// of the last one stay in flight across it (__syncthreads() would wait for them).
__device__ __forceinline__ void lds_barrier_f() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#ifdef EVO_TRACE
// a cycle count per phase and wave for EVO_TRACE_ROWS rows of every workgroup's chunk, from its fifth row on
#define EVO_TRACE_ROWS 8
#define EVO_TR(slot)                                                                             \
    do {                                                                                         \
        if (e.trace && (threadIdx.x & 63) == 0 && t >= 4 && t < 4 + EVO_TRACE_ROWS)              \
            e.trace[(((int64_t)blockIdx.x * 8 + (threadIdx.x >> 6)) * EVO_TRACE_ROWS + (t - 4)) * 16 + (slot)] = clock64(); \
    } while (0)
#else
#define EVO_TR(slot) do {} while (0)
#endif

// acc + the sum of the eight 16-bit values of x, two per instruction.
template <typename T>
__device__ __forceinline__ float pair_sums(typename Mfma<T>::v8 x, float acc) {
    typename Mfma<T>::v8 one;
#pragma unroll
    for (int i = 0; i < 8; ++i) one[i] = (T)1.0f;
    return dot8<T>(x, one, acc);
}

// The copy of a wave's 32 bias rows (256 keys, 16 bits each) that rows of unaligned length pass through: rows
// 16 bytes further apart than their length, so that the 16-byte pieces of different rows fall into different banks.
constexpr int kBiasCopyPitch = 256 * 2 + 16;
constexpr int kBiasCopyBytes = 8 * 32 * kBiasCopyPitch;
// whether every bias row starts on a 16-byte boundary and is a whole number of 16-byte pieces long
static __host__ __device__ inline bool fwdr_rows16(const EvoAttnParams &p) {
    return p.N % 8 == 0 && ((uintptr_t)p.bias & 15) == 0 && p.bias_stride_b % 8 == 0 && p.bias_stride_h % 8 == 0 &&
           p.bias_stride_row % 8 == 0;
}

// BIASK: 0 no bias, 1 fp32 tiles (x log2(e), accumulator order) as C operands, 2 the caller's 16-bit rows through the identity
// GATED: the output gate in the epilogue (kernels of their own: the ungated one carries none of their registers);
// 1: the gate's logits asked for in the epilogue, 2: copied into LDS while the row is computed (see gate_dma below)
template <typename T, int D, int BIASK, int GATED>
__global__ void __launch_bounds__(512) mfma_fwd_ring(EvoAttnParams p, Extra e) {
    typedef FwdRingGeo<D> R;
    constexpr int C = R::C;
    constexpr int KSD = (D + 15) / 16;             // data k-steps
    constexpr bool AUG_IN_PAD = D == 8;            // mask columns share k-step 0 with the data
    constexpr int KS = AUG_IN_PAD ? 1 : KSD + 1;
    constexpr int DT = (D + 31) / 32;
    constexpr bool RESID = D <= 16;
    constexpr float TAU = 8.0f;
    constexpr int IPW = (R::I_ALL + 7) / 8;        // most pieces one wave moves per stage
    typedef typename Mfma<T>::v8 v8;
    typedef typename Mfma<T>::v4 v4;

    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, g = lane >> 5;
    const int NT = (p.N + 31) / 32;
    const int np256 = (p.N + 255) / 256 * 256;
    const int nsteps = (p.N + 63) / 64;
    // Where the heads lie inside a token (the per-head layout) a cache line holds rows of several heads: the heads
    // of a chunk of S rows then run on one XCD, behind one L2 (consecutive workgroup ids go round the XCDs).
    const unsigned wid = p.stride_h < p.stride_n ? xcd_remap(blockIdx.x, gridDim.x) : blockIdx.x;
    const unsigned bh = wid % (unsigned)(p.B * p.H);
    const int c = wid / (unsigned)(p.B * p.H);
    const int b = bh / p.H, h = bh % p.H;
    const int q0 = wave * 32;
    const bool qact = q0 < p.N;
    const int qrow = min(q0 + li, p.N - 1);
    const int64_t sn = p.stride_n;
    const float cscale = p.scale * kLog2e;

    // bias of this wave's query rows, as B operands: lane = query li, k-step (j, ks) holds keys
    // 32 j + 16 ks + 8 g .. + 7
    v8 bres[BIASK == 2 ? 16 : 1];
    f32x16 btile[BIASK == 1 ? 8 : 1];
    if (BIASK == 1) {
        const int bb = e.bias_batches > 1 ? b : 0;
        // (tiles of a bias in the dtype of q are prepared as given, 16 bits per entry: log2 units here)
        const int64_t tile0 = ((((int64_t)bb * p.H + h) * NT + min(wave, NT - 1)) * NT) * 1024 + lane * 16;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int64_t o = tile0 + (int64_t)min(j, NT - 1) * 1024;
            if (e.bq16) {   // uniform
                Tile16 t;
                load_tile16(e.bq16 + o, t);
                unpack_tile16<T>(t, kLog2e, btile[j]);
            } else {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(e.bq + o + 4 * rr);
                    btile[j][4 * rr] = v[0]; btile[j][4 * rr + 1] = v[1]; btile[j][4 * rr + 2] = v[2]; btile[j][4 * rr + 3] = v[3];
                }
            }
        }
    }
    // the identity as A operands: row = key li of the tile, column 16 ks + 8 g + i
    v8 idh[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i) idh[ks][i] = (T)(li == 16 * ks + 8 * g + i ? 1.0f : 0.0f);
    if (BIASK == 2) {
        const int bb = e.bias_batches > 1 ? b : 0;
        const T *brow = (const T *)p.bias + (int64_t)bb * p.bias_stride_b + (int64_t)h * p.bias_stride_h +
                        (int64_t)qrow * p.bias_stride_row;
        // Rows that start on 16-byte boundaries are read in 16-byte pieces.  Other rows (a row length that is no
        // multiple of 8) go through LDS once per workgroup: every wave copies its 32 rows with the lanes along the
        // row (coalesced 2-byte loads; a lane per row would touch 64 cache lines per load) and takes its pieces from
        // there.  The copy lies where the stages will (and beyond: the launcher asks for kBiasCopyBytes of LDS for
        // such rows), so a barrier separates the last read from the first stage.
        const bool rows16 = fwdr_rows16(p);   // uniform
        if (rows16) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                // chunks past the row repeat its last one (those keys carry the mask floor)
                const int key0 = (j >> 1) * 32 + 16 * (j & 1) + 8 * g;
                bres[j] = ld8(brow + min(key0, p.N - 8));
            }
        } else {
            unsigned char *wb = lds + wave * (32 * kBiasCopyPitch);
            const T *bmat = (const T *)p.bias + (int64_t)bb * p.bias_stride_b + (int64_t)h * p.bias_stride_h;
            for (int r = 0; r < 32; ++r) {
                const T *row = bmat + (int64_t)min(q0 + r, p.N - 1) * p.bias_stride_row;
#pragma unroll
                for (int cc = 0; cc < 4; ++cc) {
                    const int key = cc * 64 + lane;   // keys past the row repeat its last one
                    *reinterpret_cast<T *>(wb + r * kBiasCopyPitch + key * 2) = row[min(key, p.N - 1)];
                }
            }
            // (LDS serves a wave's accesses in order; the fence keeps the compiler from moving the reads up)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int key0 = (j >> 1) * 32 + 16 * (j & 1) + 8 * g;
                bres[j] = *reinterpret_cast<const v8 *>(wb + li * kBiasCopyPitch + key0 * 2);
            }
            __syncthreads();
        }
    }

    const int s_begin = c * e.chunk, s_end = min(p.S, s_begin + e.chunk);
    const int nrows = s_end - s_begin;
    if (nrows <= 0) return;   // uniform over the workgroup
    // element offset of row 0 of problem (b, h, s_begin); S row s is (s - s_begin) * stride_s on
    const int64_t base0 = (int64_t)b * p.stride_b + (int64_t)h * p.stride_h + (int64_t)s_begin * p.stride_s;
    // where the gated form's copy of the gate logits lies: behind the stages (and the bias rows' copy where that is used)
    constexpr int kStageMost = BIASK == 2 && R::LDS_BYTES < kBiasCopyBytes ? kBiasCopyBytes : R::LDS_BYTES;
    const int gate_off = BIASK == 2 && !fwdr_rows16(p) ? kStageMost : R::LDS_BYTES;
    // Taken where a head's rows lie apart (heads inside a token: 8-byte pieces of 2 D bytes out of every row of
    // the tensor; gated forward at S = 512, N = 256, H = 8, head dim 32: 144 against 157 us); where they lie one
    // after the other the loads from the epilogue are as fast or faster (133 against 137 us).  Two kernels: one
    // kernel with both ways spills more and runs the second case at 144 us.
    constexpr bool gate_dma = GATED == 2;

    // ---- the stage of row s_begin + t lives in buffer t & 1.  It is a list of 1 KB pieces
    // (64 lanes x 16 bytes): K, V, then the mask columns; piece n belongs to wave n % 8.  Lane
    // i of piece m of K or V fills LDS slot 64 m + i of that block, which the swizzle assigns
    // to some chunk of some row.
    u32x4 stg[IPW];
    // K and V pieces are buffer loads: a resource (in scalar registers) that describes the K or V rows of
    // the S row asked for next, one lane offset that every K and V piece shares (a piece is 64 / C rows
    // of C 16-byte chunks; the swizzle depends on the row inside the piece only), and the piece's own
    // offset, also scalar.  Rows at or beyond N lie past the end of the resource and read as zero (such
    // keys carry the mask floor), so no lane clamps its row.  The mask columns are padded to 256 keys
    // and come by plain loads.  In LDS piece n lies at n KB, whatever its kind.
    static_assert(R::K_BYTES == R::I_K * 1024 && R::OFF_A == 2 * R::I_K * 1024, "piece n of a stage lies at n KB");
    static_assert(C == 1 || C == 2 || C == 4, "one lane offset for every K and V piece needs a head dim of 8, 16 or 32");
    const int kv_valid = (int)(((int64_t)(p.N - 1) * sn + D) * 2);   // bytes from a problem's first K (V) row to the end of its last
    const unsigned kv_voff = (unsigned)((lane / C) * (int)sn * 2 + (((lane % C) ^ (((lane / C) / R::RPB) % C)) << 4));
    const int kv_piece = (64 / C) * (int)sn * 2;                     // bytes from one K (V) piece to the next
    // of the row that is asked for next (they stay at the chunk's last row)
    const unsigned char *krow = reinterpret_cast<const unsigned char *>((const T *)p.k + base0);
    const unsigned char *vrow = reinterpret_cast<const unsigned char *>((const T *)p.v + base0);
    const unsigned char *arow = reinterpret_cast<const unsigned char *>(e.m2a + ((int64_t)b * p.S + s_begin) * np256);
    int frow = 0;
    auto fetch_row = [&](int t) {   // moves the pointers to row min(t, nrows - 1); t grows by at most one per call
        if (t > frow && t < nrows) {
            krow += p.stride_s * 2;
            vrow += p.stride_s * 2;
            arow += (int64_t)np256 * 16;
            frow = t;
        }
    };
    // Loads are unconditional (the row past the end repeats the last row, a wave with fewer pieces
    // repeats a mask piece) so that the staging registers stay registers.
    auto fetch_piece = [&](int i) {
        const int n = wave + 8 * i;   // uniform
        if (n < 2 * R::I_K) {
            const bool isv = n >= R::I_K;
            const int m = isv ? n - R::I_K : n;
            const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void *)(isv ? vrow : krow), 0, kv_valid, 0x00020000);
            stg[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)kv_voff, m * kv_piece, 0);
        } else {
            const int m = min(n, R::I_ALL - 1) - 2 * R::I_K;
            stg[i] = *reinterpret_cast<const u32x4 *>(arow + m * 1024 + lane * 16);
        }
    };
    auto fetch = [&](int t) {
        fetch_row(t);
#pragma unroll
        for (int i = 0; i < IPW; ++i) fetch_piece(i);
    };
    const int lds_piece0 = wave * 1024 + lane * 16;   // where this lane's 16 bytes of the wave's first piece lie in a stage
    auto stash = [&](int t) {
        if (t >= nrows) return;
        unsigned char *buf = lds + (t & 1) * R::BUF_BYTES + lds_piece0;
#pragma unroll
        for (int i = 0; i < IPW; ++i)
            if (wave + 8 * i < R::I_ALL) *reinterpret_cast<u32x4 *>(buf + i * 8192) = stg[i];
    };
    // this lane's half of its query row, straight from global memory
    v8 qraw[KSD], qnext[KSD];
    auto fetch_q = [&](int t, v8 (&dst)[KSD]) {
        t = min(t, nrows - 1);
        const T *Q = (const T *)p.q + base0 + (int64_t)t * p.stride_s + (int64_t)qrow * sn;
#pragma unroll
        for (int ks = 0; ks < KSD; ++ks) {
            const int ch = 2 * ks + g;
            dst[ks] = ld8(Q + (ch < C ? ch : 0) * 8);
        }
    };

    fetch(0);
    fetch_q(0, qraw);
    stash(0);

    for (int t = 0; t < nrows; ++t) {
        const int s = s_begin + t;
        const unsigned pid = bh * (unsigned)p.S + s;
        const bool dead = uniform_load(e.dead + b * p.S + s) != 0;
        EVO_TR(0);
        lds_barrier_f();   // the stage of this row is in LDS; everybody is done with the row before
        EVO_TR(1);
        const unsigned char *buf = lds + (t & 1) * R::BUF_BYTES;
        if constexpr (GATED) {
            // The gate logits of the wave's own 32 query rows go to LDS by the load path itself (16 bytes per lane,
            // lane L to L * 16 of the wave's piece, no register in between) while the row is computed: asked for in
            // the epilogue they were waited for with nothing else to do, and asked for earlier into registers they
            // cost registers the kernel does not have.  The wave alone writes and reads its piece.
            if (qact && gate_dma) {
#pragma unroll
                for (int i = 0; i < kGatePieces<D>; ++i) {
                    const int L = i * 64 + lane, row = min(L / C, 31), ch = L % C;
                    const T *src = (const T *)p.gate + base0 + (int64_t)t * p.stride_s + (int64_t)min(q0 + row, p.N - 1) * sn + ch * 8;
                    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                                     (__attribute__((address_space(3))) void *)(lds + gate_off + wave * kGateWaveBytes<D> + i * 1024),
                                                     16, 0, 0);
                }
            }
        }

        // m: the maximum the probabilities are relative to; mf: what the mask k-step currently
        // subtracts inside the MFMA (m, or 0 while m is not yet known or too large to be
        // carried in three 16-bit columns next to scores of order one)
        float m = 0.0f, mf = 0.0f, l = 0.0f;
        f32x16 oacc[DT];
        if (qact) {
            v8 qf[KSD], qlo[KSD];
            const float cq = dead ? 0.0f : cscale;
            const float bscale = dead ? 0.0f : kLog2e;
#pragma unroll
            for (int ks = 0; ks < KSD; ++ks) {
                qf[ks] = zero8<T>();
                qlo[ks] = zero8<T>();
                if (2 * ks + g < C) scaled_hilo8<T>(qraw[ks], cq, qf[ks], qlo[ks]);
            }
            v8 qaug = aug8<T>(ones3<T>(), uint2{0u, 0u});   // ones x mask columns, -mf x ones
            v8 qaug_hi0 = g ? zero8<T>() : qaug;             // the same as a whole k-step: zeros in the upper half
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.0f;

            // ---- scores of one 64-key step: S^T = bias^T log2(e) + K Q^T + mask - mf
            auto scores = [&](int step, f32x16 &a0, f32x16 &a1) {
                const int kb = step * 64;
                bool started = false;
                if (BIASK == 2) {
                    f32x16 z;
#pragma unroll
                    for (int r = 0; r < 16; ++r) z[r] = 0.0f;
                    // the bias tile itself through the matrix core (exact: one product per
                    // element), then into log2 units in fp32; a scaled identity would need a hi
                    // and a lo part of the constant, twice the MFMAs
                    a0 = Mfma<T>::mma(idh[0], bres[4 * step], z);
                    a1 = Mfma<T>::mma(idh[0], bres[4 * step + 2], z);
                    a0 = Mfma<T>::mma(idh[1], bres[4 * step + 1], a0);
                    a1 = Mfma<T>::mma(idh[1], bres[4 * step + 3], a1);
                    // (a row with every key masked takes no bias: the factor is 0 there)
#pragma unroll
                    for (int r = 0; r < 16; ++r) a0[r] *= bscale;
#pragma unroll
                    for (int r = 0; r < 16; ++r) a1[r] *= bscale;
                    started = true;
                }
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    v8 k0, k1, qb;
                    if (ks < KSD) {
                        const int ch = 2 * ks + g;
                        if (AUG_IN_PAD && g == 1) {
                            k0 = *reinterpret_cast<const v8 *>(buf + R::OFF_A + (kb + li) * 16);
                            k1 = *reinterpret_cast<const v8 *>(buf + R::OFF_A + (kb + 32 + li) * 16);
                            qb = qaug;
                        } else {
                            k0 = *reinterpret_cast<const v8 *>(buf + R::swz(kb + li, ch < C ? ch : 0));
                            k1 = *reinterpret_cast<const v8 *>(buf + R::swz(kb + 32 + li, ch < C ? ch : 0));
                            qb = qf[ks];
                        }
                    } else {
                        // the mask k-step: its columns sit in the lower half (lane group 0).  The
                        // upper half of the Q side is zero, so the upper half of the K side may hold
                        // any finite values: both lane groups read the same chunk (no registers to
                        // clear, no exec mask to change per step)
                        k0 = *reinterpret_cast<const v8 *>(buf + R::OFF_A + (kb + li) * 16);
                        k1 = *reinterpret_cast<const v8 *>(buf + R::OFF_A + (kb + 32 + li) * 16);
                        qb = qaug_hi0;
                    }
                    if (ks == 0 && BIASK == 1 && !dead) {  // uniform
                        a0 = Mfma<T>::mma(k0, qb, btile[2 * step]);
                        a1 = Mfma<T>::mma(k1, qb, btile[2 * step + 1]);
                    } else if (ks == 0 && !started) {
                        f32x16 z;
#pragma unroll
                        for (int r = 0; r < 16; ++r) z[r] = 0.0f;
                        a0 = Mfma<T>::mma(k0, qb, z);
                        a1 = Mfma<T>::mma(k1, qb, z);
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
            };
            // ---- online softmax of one step, part 1: where the maximum stands.  `used` is the
            // mf the step's scores were formed with (they are relative to it).
            auto settle = [&](int step, f32x16 &a0, f32x16 &a1, float used) {
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
                const bool grow = step == 0 || cand > m + TAU;
                if (__any(grow || m != used)) {
                    const float mn = grow ? cand : m;
                    if (step != 0) {
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
                    qaug = aug8<T>(ones3<T>(), pack_split3<T>(-mf));
                    qaug_hi0 = g ? zero8<T>() : qaug;
                }
            };
            // ---- part 2: P = exp2, rounded to T, and this lane's sum of the rounded values
            auto probs = [&](f32x16 &a0, f32x16 &a1, v8 (&pf)[4], float &ls) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    a0[r] = fast_exp2(a0[r]);
                    a1[r] = fast_exp2(a1[r]);
                }
                ls = 0.0f;
#pragma unroll
                for (int ts = 0; ts < 4; ++ts) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) pf[ts][i] = (T)((ts < 2 ? a0 : a1)[8 * (ts & 1) + i]);
                    ls = pair_sums<T>(pf[ts], ls);
                }
            };
            // ---- part 3: O^T += V^T P^T with V^T fragments by transposing reads of row-major V
            auto weigh = [&](int step, const v8 (&pf)[4], float ls) {
                const int kb = step * 64;
                l += ls;
#pragma unroll
                for (int ts = 0; ts < 4; ++ts) {
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        // lanes whose column lies past the head dim (rows of the product that are never stored; a row of the
                        // product depends on its own row of this operand only) read column 0 instead of being masked and cleared
                        const int col0 = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
                        const int col = (D % 32 == 0 || col0 < D) ? col0 : 0;
                        v8 va;
#pragma unroll
                        for (int h2 = 0; h2 < 2; ++h2) {
                            const int row = kb + 16 * ts + 8 * h2 + 4 * g + ((lane & 15) >> 2);
                            const unsigned char *ad = buf + R::OFF_V + R::swz(row, col >> 3) + (col & 7) * 2;
                            s16x4 rd = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                (s16x4 __attribute__((address_space(3))) *)ad);
                            v4 rv = __builtin_bit_cast(v4, rd);
                            va[4 * h2] = rv[0]; va[4 * h2 + 1] = rv[1]; va[4 * h2 + 2] = rv[2]; va[4 * h2 + 3] = rv[3];
                        }
                        oacc[dt] = Mfma<T>::mma(va, pf[ts], oacc[dt]);
                    }
                }
            };
            // (A second score set, so that the matrix core could form the scores of step s+1 under
            // the softmax of step s, does not fit 256 registers next to the resident bias: the
            // spilled form measured 153 us against 120 us at S = 512, N = 256, H = 8.)
            f32x16 sa0, sa1;
#pragma unroll
            for (int step = 0; step < 4; ++step) {
                EVO_TR(2 + step);
                // The two waves of a SIMD (w and w + 4) take turns at the higher issue priority, step by
                // step: left alone the older wave is always served first, ends its row a quarter of a
                // row early and waits at the barrier while the younger one runs on alone.
                if (((step ^ (wave >> 2)) & 1) != 0) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
                {
                    // The next row's requests go out a few per step rather than all after the
                    // barrier: eight waves asking at once queue up behind the CU's load path
                    // (16 clocks per request), and the last in line start their row late.
                    constexpr int PPS = (IPW + 2) / 3;
                    if (step == 0) fetch_row(t + 1);
#pragma unroll
                    for (int i = step * PPS; i < (step + 1) * PPS && i < IPW; ++i)
                        if (step < 3) fetch_piece(i);
                    if (step == 2) fetch_q(t + 1, qnext);
                }
                if (step < nsteps) {  // uniform
                    const float used = mf;
                    scores(step, sa0, sa1);
                    v8 pf[4];
                    float ls;
                    // After the first step the scores come out of the MFMA relative to m already
                    // (where m fits the mask columns): the step skips the search for its maximum
                    // and looks at the sums instead.  A lane sum beyond 2^13 (or not a number)
                    // means some score stands far above m: the step is then redone the long way.
                    bool settled = step != 0 && !__any(m != used);
                    if (settled) {
                        probs(sa0, sa1, pf, ls);
                        if (__any(!(ls <= 8192.0f))) {
                            settled = false;
                            scores(step, sa0, sa1);
                        }
                    }
                    if (!settled) {
                        settle(step, sa0, sa1, used);
                        probs(sa0, sa1, pf, ls);
                    }
                    weigh(step, pf, ls);
                }
            }

        }
        else {
            fetch(t + 1);
            fetch_q(t + 1, qnext);
        }
        // The next stage goes into the other buffer, free since the barrier above.  This comes
        // before the row's own stores: what waits for the staged loads must not have the
        // stores in front of it (vector memory operations complete in order).
        EVO_TR(6);
        stash(t + 1);
        EVO_TR(7);
        if (qact) {
            {   // the two lane groups hold the two halves of each query's sum
                const unsigned u = __float_as_uint(l);
                auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                l = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
            }
            const float inv = 1.0f / l;
            const int q = q0 + li;
            if (q < p.N) {
                T *O = (T *)p.o + base0 + (int64_t)t * p.stride_s + (int64_t)q * sn;
                if (g == 0) p.lse[(int64_t)pid * p.N + q] = (m + __log2f(l)) * kLn2;
                if (!GATED || p.o) {   // uniform (with a gate the caller may ask for the gated output alone)
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) store_row_tile<T>(O, dt * 32, D, oacc[dt], inv, g);
                }
                if constexpr (GATED) {   // sigmoid(gate) * O goes out as a second tensor, from the same registers
                    const int64_t off = base0 + (int64_t)t * p.stride_s + (int64_t)q * sn;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) oacc[dt][r] *= inv;
                        // the wave's piece of the gate, in LDS since the top of the row (the compiler does not
                        // order the reads after that copy by itself)
                        if (gate_dma) {
                            if (dt == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                            gate_row_tile<T>((const T *)(lds + gate_off + wave * kGateWaveBytes<D>) + li * D, dt * 32, D, oacc[dt], g);
                        } else {
                            gate_row_tile<T>((const T *)p.gate + off, dt * 32, D, oacc[dt], g);
                        }
                        store_row_tile<T>((T *)p.o_gated + off, dt * 32, D, oacc[dt], 1.0f, g);
                    }
                }
            }
        }
        EVO_TR(8);
#pragma unroll
        for (int ks = 0; ks < KSD; ++ks) qraw[ks] = qnext[ks];
    }
}

// ------------------------------------------------------------------ launcher

template <typename T, int D, int BIASK, int GATED>
static int fwdr_launch_g(const EvoAttnParams &p, const Extra &e0, hipStream_t st) {
    typedef FwdRingGeo<D> R;
    static PerDevice done{};
    int cus = 256;
    auto kern = mfma_fwd_ring<T, D, BIASK, GATED>;
    constexpr int LDS_MOST = BIASK == 2 && R::LDS_BYTES < kBiasCopyBytes ? kBiasCopyBytes : R::LDS_BYTES;
    if (const int rc = ensure_dynamic_lds((const void *)kern, LDS_MOST + (GATED == 2 ? kGateBytes<D> : 0), done, &cus)) return rc;
    const int lds_bytes = (BIASK == 2 && !fwdr_rows16(p) ? LDS_MOST : R::LDS_BYTES) + (GATED == 2 ? kGateBytes<D> : 0);
    // one workgroup per CU: chunks of S rows such that (b, h, chunk) items about fill the chip
    Extra e = e0;
    const int bh = p.B * p.H;
    const int want = chunks_for_rounds(bh, p.S, cus, 0.0);
    e.chunk = (p.S + want - 1) / want;
    e.n_chunks = (p.S + e.chunk - 1) / e.chunk;
    kern<<<(unsigned)bh * (unsigned)e.n_chunks, 512, lds_bytes, st>>>(p, e);
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

template <typename T, int D, int BIASK>
static int fwdr_launch(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    if (!p.gate) return fwdr_launch_g<T, D, BIASK, 0>(p, e, st);
    return p.stride_h < p.stride_n ? fwdr_launch_g<T, D, BIASK, 2>(p, e, st) : fwdr_launch_g<T, D, BIASK, 1>(p, e, st);
}

// whether the form with resident fp32 bias tiles keeps them in registers (the dispatch in api.hip sends an
// fp32 bias here under the same condition)
static bool fwdr_tiles_fit(const EvoAttnParams &p) { return EVO_D == 8 && !p.gate; }

template <typename T>
static int fwdr_bias(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    if (p.bias_dtype == EVO_NONE) return fwdr_launch<T, EVO_D, 0>(p, e, st);
    // Two resident forms.  fp32 tiles as C operands (128 registers) fit the register file only at head dim 8
    // without a gate, and are the faster form there (S = 1024, N = 256, H = 8: 119 against 143 us; N = 201, S = 512:
    // 64 against 85 us), also for an fp32 bias.  Elsewhere they spill 77..169 registers (head dim 16, N = 256: 170
    // against 82 us) and a bias in the dtype of q stays resident as the caller's 16-bit rows (64 registers); an
    // fp32 bias is then served by the one-workgroup-per-problem forward (the dispatch sends none here).
    // EVO_FLAG_DEBUG_FWD_BIAS_TILES selects the fp32 tiles wherever the kernel runs, for comparison.
    const bool tiles = fwdr_tiles_fit(p) || p.bias_dtype != p.dtype || (p.flags & EVO_FLAG_DEBUG_FWD_BIAS_TILES);
    return tiles ? fwdr_launch<T, EVO_D, 1>(p, e, st) : fwdr_launch<T, EVO_D, 2>(p, e, st);
}

// Largest N this kernel takes for the head dim (0: not built for it).
int EVO_CAT(mfma_fwdr_max_n_d, EVO_D)() { return EVO_D <= 32 ? 256 : 0; }   // 64: the resident tiles do not fit the registers

int EVO_CAT(launch_mfma_fwdr_d, EVO_D)(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
#if EVO_D <= 32
    return p.dtype == EVO_BF16 ? fwdr_bias<bf16_t>(p, e, st) : fwdr_bias<f16_t>(p, e, st);
#else
    (void)p; (void)e; (void)st;   // (no kernel is built: the resident bias does not fit the registers at this width)
    return EVO_EUNSUPPORTED;
#endif
}

}  // namespace evo
