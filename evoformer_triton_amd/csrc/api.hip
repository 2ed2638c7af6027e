// C ABI of the library: parameter validation, workspace layout and kernel dispatch.
// Everything in this file runs on the host; nothing here needs a GPU except the two
// enqueue entry points.
#include <atomic>

#include "common.h"
#include "kernels.h"

// Prepared operands of evoattn_fwd_static: one array per GPU the library runs on, held until the
// process ends.  In host code the name stands for the symbol only; the array's device address is
// asked for once per device (static_prep below) and only that address is handed to kernels.
static __device__ __align__(256) unsigned char scratch[EVOATTN_STATIC_PREP_BYTES];

namespace evo {

static inline size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }
static inline bool aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }
static inline int elem_size(int dtype) { return dtype == EVO_F32 ? 4 : 2; }


// Elements from the first to one past the last element of a q-family tensor (= B*H*S*N*D when it is dense).
static int64_t q_span(const EvoAttnParams &p) {
    const int64_t st4[4] = {p.stride_b, p.stride_h, p.stride_s, p.stride_n};
    const int64_t ext[4] = {p.B, p.H, p.S, p.N};
    int64_t span = p.D;
    for (int i = 0; i < 4; ++i) span += (ext[i] - 1) * st4[i];
    return span;
}

static int check_common(const EvoAttnParams *p) {
    if (!p) return EVO_EINVAL;
    if (p->B <= 0 || p->S <= 0 || p->N <= 0 || p->H <= 0 || p->D <= 0) return EVO_EINVAL;
    if (p->dtype != EVO_BF16 && p->dtype != EVO_F16 && p->dtype != EVO_F32) return EVO_EINVAL;
    if (p->bias_dtype != EVO_NONE && p->bias_dtype != EVO_F32 && p->bias_dtype != p->dtype) return EVO_EINVAL;
    if (p->mask_kind < EVO_MASK_NONE || p->mask_kind > EVO_MASK_F16) return EVO_EINVAL;
    if ((p->bias_dtype == EVO_NONE) != (p->bias == nullptr)) return EVO_EINVAL;
    if ((p->mask_kind == EVO_MASK_NONE) != (p->mask == nullptr)) return EVO_EINVAL;
    if (!p->q || !p->k || !p->v || !p->lse) return EVO_EINVAL;
    // (with a gate the gated output may stand alone: the forward then writes no ungated O and the backward,
    // whose gate pass forms delta from the gated output, reads none)
    if (!p->o && !(p->gate && p->o_gated)) return EVO_EINVAL;
    if (!(p->scale == p->scale) || p->scale <= 0.0f) return EVO_EINVAL;
    if (p->flags & ~EVO_FLAG_ALL) return EVO_EINVAL;
    // (a second call on the same dout would apply the gate to it a second time)
    if ((p->flags & EVO_FLAG_GATE_DOUT_INPLACE) && (p->flags & (EVO_FLAG_ONLY_DQ | EVO_FLAG_ONLY_DKDV))) return EVO_EINVAL;
    if (p->gate) {
        // The gate is read and its products written element for element like q; the backward keeps the gradient
        // of the ungated output in the workspace, laid out like q, gaps included: the q-family may be dense or a
        // slot of a buffer of up to 8 such tensors (Q, K, V and the gate as one projection's result), not sparser.
        if (p->D % 8 || p->H > 256) return EVO_EUNSUPPORTED;   // (the gate's backward pass keeps 128 bytes of LDS per head)
        if (q_span(*p) > 8 * (int64_t)p->B * p->H * p->S * p->N * p->D) return EVO_EUNSUPPORTED;
    } else if (p->o_gated || p->dgate) {
        return EVO_EINVAL;
    }
    if (p->D != 8 && p->D != 16 && p->D != 32 && p->D != 64 && p->D != 128) return EVO_EUNSUPPORTED;
    if (p->stride_b < 0 || p->stride_h < 0 || p->stride_s < 0 || p->stride_n < p->D) return EVO_EINVAL;
    if (p->bias && (p->bias_stride_b < 0 || p->bias_stride_h < 0 || p->bias_stride_row < p->N)) return EVO_EINVAL;
    if (p->mask && (p->mask_stride_b < 0 || p->mask_stride_s < 0)) return EVO_EINVAL;
    // index ranges: problems and rows are 32-bit in the kernels, element offsets 64-bit
    const int64_t probs = (int64_t)p->B * p->H * p->S;
    if (probs > (int64_t)1 << 26 || (int64_t)p->N > (int64_t)1 << 20) return EVO_EOVERFLOW;
    if (probs * ((p->N + 31) / 32) > (int64_t)0x7fffffff) return EVO_EOVERFLOW;
    if ((int64_t)p->B * p->H * p->N * ((p->N + 63) / 64) > (int64_t)0x7fffffff) return EVO_EOVERFLOW;
    const int es = elem_size(p->dtype);
    if (!aligned(p->q, es) || !aligned(p->k, es) || !aligned(p->v, es) || !aligned(p->o, es) || !aligned(p->lse, 4))
        return EVO_EALIGN;
    if (p->bias && !aligned(p->bias, elem_size(p->bias_dtype))) return EVO_EALIGN;
    if (p->gate) {
        // The gate's kernels move rows in 8- and 16-byte pieces whichever attention kernels run: every tensor laid out
        // like q starts on a 16-byte boundary and every stride is a whole number of such pieces (o_gated may be NULL
        // in a backward call, o in any call).
        const int64_t per16 = 16 / es;
        if (p->stride_b % per16 || p->stride_h % per16 || p->stride_s % per16 || p->stride_n % per16) return EVO_EALIGN;
        if (!aligned(p->gate, 16) || !aligned(p->o_gated, 16) || !aligned(p->o, 16)) return EVO_EALIGN;
    }
    if (p->mask_kind == EVO_MASK_F32 && !aligned(p->mask, 4)) return EVO_EALIGN;
    if ((p->mask_kind == EVO_MASK_BF16 || p->mask_kind == EVO_MASK_F16) && !aligned(p->mask, 2)) return EVO_EALIGN;
    return EVO_OK;
}

// The matrix-core kernels read rows with 16-byte loads and keep one 32-wide key tile per
// 16 accumulator registers in the dBias kernel (at most 16 tiles per wave, 4 waves).
static bool long_rows_bwd_ok(const EvoAttnParams &p);
static bool mfma_ok(const EvoAttnParams &p, int pass) {
    if (p.flags & EVO_FLAG_FORCE_GENERIC) return false;
    if (p.dtype != EVO_BF16 && p.dtype != EVO_F16) return false;
    if (p.D != 8 && p.D != 16 && p.D != 32 && p.D != 64 && p.D != 128) return false;
    if (p.stride_b % 8 || p.stride_h % 8 || p.stride_s % 8 || p.stride_n % 8) return false;
    // (the kernels address the rows of one (b, h, s) problem by 32-bit byte offsets from its first row, also the rows
    // up to the next multiple of 256 beyond N, which their buffer loads must find out of range rather than wrapped)
    if (((int64_t)(p.N + 511) * p.stride_n + p.D) * 2 >= ((int64_t)1 << 31)) return false;
    if (!aligned(p.q, 16) || !aligned(p.k, 16) || !aligned(p.v, 16) || !aligned(p.o, 16)) return false;
    if (pass == EVO_PASS_BWD) {
        if (p.N > 2048 && !long_rows_bwd_ok(p)) return false;
        if (!aligned(p.dout, 16) || !aligned(p.dq, 16) || !aligned(p.dk, 16) || !aligned(p.dv, 16)) return false;
    }
    return true;
}

static int bias_vec_ok(const EvoAttnParams &p) {
    if (!p.bias) return 0;
    const size_t a = p.bias_dtype == EVO_F32 ? 16 : 8;
    return aligned(p.bias, a) && p.bias_stride_b % 4 == 0 && p.bias_stride_h % 4 == 0 && p.bias_stride_row % 4 == 0;
}

// The prepared bias tiles (two copies in accumulator order, fp32 or, for a bias in the dtype of q,
// 16 bits per entry) cost 6 to 12 bytes of memory traffic per bias entry before any kernel has
// used one; each kernel then reads 2 or 4 bytes per entry and S row.  With very few S rows per (batch, head) - the reference's own speed benchmark has one -
// the one-workgroup-per-problem kernels read the caller's tensor instead, which needs rows that
// allow 16-byte (fp32) or 8-byte loads.  EVO_FLAG_DEBUG_BIAS_TILES keeps the tiles, for comparison.
static bool bias_direct(const EvoAttnParams &p) {
    if (!p.bias || p.S > 4 || (p.flags & EVO_FLAG_DEBUG_BIAS_TILES) || p.N % 4) return false;
    // The 16-bit tiles of a bias in the dtype of q are cheap to prepare (2 + 4 bytes of traffic per entry at
    // streaming rate) and pay from the first S row on where the score work per entry is small: they are taken
    // for rows beyond 256 keys unless S = 1 at head dim 64 or more (whole step, us, tiles against the caller's
    // tensor: H = 8, D = 32, N = 1024, S = 1 / 2 / 4 103 / 111 / 151 against 121 / 142 / 189; N = 2048 210 / 357 / 444
    // against 244 / 418 / 545; B = 4, H = 32, D = 64, N = 1024, S = 1 / 2 / 4 596 / 1383 / 2320 against 536 / 1528 /
    // 2718; up to 256 keys the tiles would bring the chunk-of-rows kernels, which need more S rows: 49 against
    // 40 us at S = 4).  An fp32 bias keeps the direct reads up to 4 rows (S = 1: 257 against 140 us).
    if (p.bias_dtype == p.dtype && p.dtype != EVO_F32 && p.N > 256 && !(p.S == 1 && p.D >= 64)) return false;
    // beyond 2048 keys a dBias summed over several S rows needs the kernel that reads prepared tiles
    // (decided without looking at dbias: the forward, which prepares, has none)
    if (p.N > 2048 && p.S > 1) return false;
    if (p.bias_dtype != EVO_F32 && p.bias_dtype != p.dtype) return false;
    if ((int64_t)p.N * p.bias_stride_row >= ((int64_t)1 << 31)) return false;   // 32-bit offsets inside one (b, h) matrix
    return bias_vec_ok(p) != 0;
}

// The dQ kernel that double-buffers its operands in LDS takes rows of limited length.
static bool dq_ring_ok(const EvoAttnParams &p) {
    return !(p.flags & EVO_FLAG_PER_PROBLEM) && !bias_direct(p) && mfma_dqr_qrows(p.D, p.N) > 0;
}

// Where dBias is not a sum over S rows (no bias, one that takes no gradient, or S = 1, where
// dBias is dS itself) nothing ties a wave of the dQ kernel to a key tile for a chunk of S rows:
// the kernel whose waves own their query rows for all keys takes those problems, and with
// S = 1 writes dBias as it goes (no partials, no reduction).  Its workgroups take 128 query
// rows each and walk over the keys one tile after the other: with very few of them the
// kernels that split a row's keys over the waves finish sooner (N = 300, 6 workgroups: 10.4 us
// against 8.2 us).  EVO_FLAG_DEBUG_NO_DQ_WIDE selects the other kernels, for comparison.
static bool dq_wide_grid_ok(const EvoAttnParams &p) {
    return !(p.flags & (EVO_FLAG_PER_PROBLEM | EVO_FLAG_DEBUG_NO_DQ_WIDE)) && (int64_t)((p.N + 127) / 128) * p.B * p.H * p.S >= 32;
}

// Long rows with a dBias to sum: either the dQ kernel over a chunk of rows, which keeps the sums of its key
// tiles next to dQ (up to 512 keys with two query tiles per workgroup or in one or two stages, beyond in
// blocks of 256 keys with one query tile), or dQ from the kernel whose waves own their query rows for all keys
// and the dBias partials from a kernel of their own that forms dS a second time.  The pair is taken where
// the one kernel has no form (beyond 768 keys; head dim 64 beyond 128 keys; head dim 8 beyond 512) and, between
// 513 and 768 keys, where the row leaves the one kernel's last 256-key block mostly empty.  Whole backward,
// bf16, H = 4, head dim 32, one kernel / the pair: N = 320 (S = 128) 92 / 110 us; N = 352, 448, 480 (S = 256)
// 177 / 190, 259 / 274, 277 / 291 us; N = 576, 704, 736 (S = 256) 459 / 436, 633 / 623, 660 / 654 us; N = 640
// (B = 2, S = 256) 1.06 / 0.99 ms; head dim 16, H = 8, S = 512: N = 576 1.51 / 1.46 ms, N = 640 1.72 / 1.63 ms,
// N = 704 2.01 / 2.06 ms.
// EVO_FLAG_DEBUG_NO_DQ_SPLIT selects the one kernel, for comparison.
static bool dq_split_ok(const EvoAttnParams &p) {
    const int min_n = p.D == 64 ? 128 : 512;
    if (p.D > 64) return false;   // the dBias kernel is not built for head dim 128
    const int rem = p.N % 256;
    const bool full_blocks = rem == 0 || rem >= (p.D == 32 ? 224 : 192);
    const bool ring = dq_ring_ok(p);
    if (full_blocks && ring) return false;
    // Fewest S rows: the second kernel's start-up has to pay.  Against the one kernel over a chunk of rows
    // (N = 768, D = 32: ahead from 8 rows on); where that kernel has no form, against the one-workgroup-per-problem
    // dQ kernel, which the pair beats from 8 rows on (bf16, dQ + dBias, us, S = 8 / 16 / 32 / 52: D = 8, H = 8, N = 768
    // 50 / 71 / 102 / 146 against 47 / 92 / 159 / 228; D = 16, N = 1024, S = 8 / 16 / 32: 53 / 84 / 152 against
    // 63 / 99 / 175; D = 64, H = 4, N = 1024, S = 16 / 32 / 59: 99 / 194 / 327 against 152 / 277 / 599; N = 300,
    // S = 16 / 32: 32 / 41 against 30 / 47), and from 1024 keys on from 2 rows (whole step, us, the pair against
    // that kernel: D = 32, H = 8, N = 1024, S = 2 / 3 / 4 / 5 / 7 108 / 113 / 114 / 149 / 159 against 110 / 131 / 150 /
    // 185 / 215; N = 2048, S = 4 / 7 331 / 600 against 444 / 826; D = 8, S = 7 472 against 730; D = 64, B = 4, H = 32,
    // N = 1024, S = 4 1.89 against 2.33 ms; at N = 640..768 with S = 5, 6 the one kernel stays ahead, 76 / 103
    // against 88 / 111).  Beyond 2048 keys that kernel has no form either.
    const int min_s = p.N >= 1024 ? 2 : !ring ? (p.D == 64 ? 16 : 8) : p.D == 32 && p.N > 512 ? 8 : 64;
    if (!p.dbias || p.S < min_s || p.N <= min_n || (p.flags & EVO_FLAG_DEBUG_NO_DQ_SPLIT) || bias_direct(p) || !dq_wide_grid_ok(p)) return false;
    return p.bias_dtype == p.dtype || p.bias_dtype == EVO_F32;   // (the dBias kernel keeps 16-bit pairs or fp32 tiles)
}

static bool dq_wide_ok(const EvoAttnParams &p) {
    return dq_wide_grid_ok(p) && (!p.dbias || p.S == 1 || dq_split_ok(p));
}
// Rows of more than 2048 keys: the dQ kernels that keep the dBias sums of a wave's key tiles in
// registers have no form that long (16 tiles per wave would be the whole register file).  The
// backward still runs on the matrix core where dQ comes from the kernel without those sums:
// no dBias asked for, S = 1, or the dBias kernel of its own (bias in the dtype of q).
static bool long_rows_bwd_ok(const EvoAttnParams &p) { return dq_wide_ok(p); }
static bool dq_writes_dbias(const EvoAttnParams &p) { return p.dbias && p.S == 1 && dq_wide_ok(p); }

// S is split into chunks; one workgroup of the dQ kernel sums dS over one chunk and
// writes one partial dBias tile.  Enough chunks to fill the chip, no more.  The kernel that
// walks over its chunk with one workgroup per CU (256 CUs) runs in rounds of 256 workgroups:
// among the chunk counts that give up to four rounds it takes the cheapest by a count of rows
// per workgroup, rounds and partials (below).
static void chunking(const EvoAttnParams &p, int *n_chunks, int *chunk) {
    const int64_t NT = (p.N + 31) / 32;
    if (dq_split_ok(p)) {
        // the dBias kernel: one workgroup per block of 128 queries x 128 keys (64 at head dim 64), (b, h) and chunk, two
        // workgroups per CU (256 CUs) at a time; among the chunk counts that give one to four rounds
        // the one that leaves the fewest slots idle in the last round (near ties: the fewest chunks)
        const int64_t kb = p.D == 64 ? 64 : 128;   // keys per block
        const int64_t base = (int64_t)((p.N + 127) / 128) * ((p.N + kb - 1) / kb) * p.B * p.H, slots = 512;
        const int64_t lo = slots / base > 0 ? slots / base : 1, hi = (4 * slots + base - 1) / base;
        int64_t want = lo;
        double best = -1.0;
        for (int64_t n = lo; n <= hi; ++n) {
            const int64_t wgs = base * n, rounds = (wgs + slots - 1) / slots;
            const double eff = (double)wgs / (double)(rounds * slots);
            if (eff > best + 0.02) { best = eff; want = n; }
        }
        if (want > p.S) want = p.S;
        *chunk = (int)((p.S + want - 1) / want);
        *n_chunks = (p.S + *chunk - 1) / *chunk;
        return;
    }
    const bool ring = dq_ring_ok(p);
    // workgroups per chunk: one per slab of query rows and head
    const int64_t base = (ring ? (p.N + mfma_dqr_qrows(p.D, p.N) - 1) / mfma_dqr_qrows(p.D, p.N) : NT) * p.B * p.H;
    int64_t want = (1024 + base - 1) / base;
    // The kernel over a chunk of rows: every chunk is a partial dBias to write and to sum again, about a
    // quarter of a row's worth (S = N = 384, H = 4 takes 10 chunks in one round of 240 workgroups over 32 in
    // three full rounds: backward 269 against 298 us; S = N = 768 8 chunks in three rounds over 5 in two:
    // 2.00 against 2.01 ms).
    if (ring) want = chunks_for_rounds(base, p.S, 256, 0.25);
    if (want < 1) want = 1;
    if (want > p.S) want = p.S;
    *chunk = (int)((p.S + want - 1) / want);
    *n_chunks = (p.S + *chunk - 1) / *chunk;
}

struct PrepLayout {
    size_t bq, bk, bq16, bk16, bt, m2, m2a, dead, total;
    int bias_batches;
};

static PrepLayout prep_layout(const EvoAttnParams &p) {
    PrepLayout w{};
    const size_t NT = (size_t)(p.N + 31) / 32;
    w.bias_batches = (p.bias && p.bias_stride_b == 0) ? 1 : p.B;
    // Bias tiles, with one extra all-zero tile at the end of each copy: for a bias in the dtype of q
    // the entries as given, 16 bits each (every kernel that reads tiles multiplies by log2 e
    // itself, in fp32: the product the fp32 tiles hold); else fp32 tiles in log2 units.
    const bool have_tiles = p.bias && !bias_direct(p);
    const bool t16_ok = have_tiles && p.bias_dtype == p.dtype && p.dtype != EVO_F32;
    const size_t tile_elems = have_tiles ? ((size_t)w.bias_batches * p.H * NT * NT + 1) * 1024 : 0;
    size_t off = 0;
    w.bq = off; off += align_up(t16_ok ? 0 : tile_elems * 4);
    w.bk = off; off += align_up(t16_ok ? 0 : tile_elems * 4);
    w.bq16 = w.bk16 = (size_t)-1;
    if (t16_ok) {
        w.bq16 = off; off += align_up(tile_elems * 2);
        w.bk16 = off; off += align_up(tile_elems * 2);
    }
    // transposed 16-bit copy for the kernel that keeps bias columns resident (the chunk-of-rows dK/dV: rows of
    // 129 keys up to its longest)
    const bool bt_ok = p.bias && !bias_direct(p) && p.bias_dtype == p.dtype && p.N % 8 == 0 && p.N > 128 &&
                       p.N <= mfma_kvr_max_n(p.D);
    w.bt = bt_ok ? off : (size_t)-1;
    if (bt_ok) off += align_up((size_t)w.bias_batches * p.H * p.N * p.N * 2);
    w.m2 = off; off += align_up((size_t)p.B * p.S * NT * 32 * 8);
    w.m2a = off; off += align_up((size_t)p.B * p.S * ((p.N + 255) / 256 * 256) * 16);
    w.dead = off; off += align_up((size_t)p.B * p.S * 4);
    w.total = off;
    return w;
}

static void fill_prep(const EvoAttnParams &p, Extra &e) {
    const PrepLayout w = prep_layout(p);
    char *base = (char *)p.prep;
    e.bias_batches = w.bias_batches;
    e.bias_direct = bias_direct(p) ? 1 : 0;
    e.bq = (float *)(base + w.bq);
    e.bk = (float *)(base + w.bk);
    e.bq16 = w.bq16 == (size_t)-1 ? nullptr : (unsigned short *)(base + w.bq16);
    e.bk16 = w.bk16 == (size_t)-1 ? nullptr : (unsigned short *)(base + w.bk16);
    e.bt = w.bt == (size_t)-1 ? nullptr : (void *)(base + w.bt);
    e.m2 = (uint2 *)(base + w.m2);
    e.m2a = (uint4 *)(base + w.m2a);
    e.dead = (int *)(base + w.dead);
    e.zero_tile = (int64_t)w.bias_batches * p.H * ((p.N + 31) / 32) * ((p.N + 31) / 32) * 1024;
}

static int check_prep(const EvoAttnParams &p) {
    if (!p.prep || p.prep_bytes < prep_layout(p).total) return EVO_EWORKSPACE;
    if (!aligned(p.prep, 256)) return EVO_EALIGN;
    return EVO_OK;
}

struct WsLayout {
    size_t delta, shift, dmask_part, dbias_part, dout_ungated, total;
    int n_chunks, chunk;
};

static WsLayout ws_layout(const EvoAttnParams &p) {
    WsLayout w{};
    const size_t rows = (size_t)p.B * p.H * p.S * p.N;
    size_t off = 0;
    w.delta = off; off += align_up(rows * 4);
    w.shift = off; off += align_up((size_t)p.B * p.S * 4);
    w.dmask_part = off; if (p.dmask) off += align_up(rows * 4);
    chunking(p, &w.n_chunks, &w.chunk);
    w.dbias_part = off;
    if (p.dbias && !dq_writes_dbias(p)) off += align_up((size_t)w.n_chunks * p.B * p.H * p.N * p.N * 4);
    w.dout_ungated = off;
    if (p.gate && !(p.flags & EVO_FLAG_GATE_DOUT_INPLACE)) off += align_up((size_t)q_span(p) * (size_t)elem_size(p.dtype));
    w.total = off;
    return w;
}

static int check_bwd(const EvoAttnParams *p) {
    if (!p->dout || !p->dq || !p->dk || !p->dv) return EVO_EINVAL;
    const int es = elem_size(p->dtype);
    if (!aligned(p->dout, es) || !aligned(p->dq, es) || !aligned(p->dk, es) || !aligned(p->dv, es)) return EVO_EALIGN;
    if (p->dbias) {
        if (p->dbias_dtype != EVO_F32 && p->dbias_dtype != p->dtype) return EVO_EINVAL;
        if (!aligned(p->dbias, elem_size(p->dbias_dtype))) return EVO_EALIGN;
    }
    if (p->dmask && !aligned(p->dmask, 4)) return EVO_EALIGN;
    if (p->gate && (!p->dgate || !aligned(p->dgate, 16) || !aligned(p->dout, 16) || !aligned(p->o, 16) || !aligned(p->o_gated, 16))) return p->dgate ? EVO_EALIGN : EVO_EINVAL;
    const WsLayout w = ws_layout(*p);
    if (!p->workspace || p->workspace_bytes < w.total) return EVO_EWORKSPACE;
    if (!aligned(p->workspace, 256)) return EVO_EALIGN;
    return EVO_OK;
}

}  // namespace evo

using namespace evo;

#ifdef EVO_TRACE
static long long *g_trace = nullptr;
extern "C" void evoattn_set_trace(void *buf) { g_trace = (long long *)buf; }
#define EVO_SET_TRACE(e) (e).trace = g_trace
#else
#define EVO_SET_TRACE(e) do {} while (0)
#endif

extern "C" {

int evoattn_version(void) { return EVOATTN_VERSION; }

const char *evoattn_strerror(int code) {
    switch (code) {
        case EVO_OK: return "ok";
        case EVO_EINVAL: return "invalid argument (null pointer, non-positive size or bad enum)";
        case EVO_EUNSUPPORTED: return "unsupported head dimension or size";
        case EVO_EALIGN: return "pointer or stride not aligned for the dtype";
        case EVO_EWORKSPACE: return "workspace missing or too small";
        case EVO_EOVERFLOW: return "extents overflow the kernels' index range";
    }
    if (code <= EVO_EHIP) return hipGetErrorString((hipError_t)(EVO_EHIP - code));
    return "unknown error";
}

int evoattn_check(const EvoAttnParams *p, int pass) {
    int rc = check_common(p);
    if (rc) return rc;
    if (pass == EVO_PASS_BWD) return check_bwd(p);
    if (pass != EVO_PASS_FWD) return EVO_EINVAL;
    if (p->gate && !p->o_gated) return EVO_EINVAL;   // the forward writes the gated output
    return EVO_OK;
}

size_t evoattn_prep_bytes(const EvoAttnParams *p) {
    if (!p || p->B <= 0 || p->S <= 0 || p->N <= 0 || p->H <= 0) return 0;
    return prep_layout(*p).total;
}

size_t evoattn_bwd_workspace_bytes(const EvoAttnParams *p) {
    if (!p || p->B <= 0 || p->S <= 0 || p->N <= 0 || p->H <= 0) return 0;
    return ws_layout(*p).total;
}

const char *evoattn_path(const EvoAttnParams *p, int pass) {
    if (!p) return "invalid";
    return mfma_ok(*p, pass) ? "mfma" : "generic";
}

// rows of 129..256 keys: a workgroup per chunk of S rows with the head's bias resident
static bool fwd_ring_ok(const EvoAttnParams &p) {
    if ((p.flags & EVO_FLAG_PER_PROBLEM) || bias_direct(p) || p.N <= 128 || p.N > mfma_fwdr_max_n(p.D)) return false;
    // Resident, a bias in the dtype of q takes 64 registers, an fp32 bias 128, which fit the register file only at
    // head dim 8 without a gate; elsewhere most of them are spilled and the one-workgroup-per-problem forward, which
    // streams the tiles, serves an fp32 bias (B = 1, S = 512, N = 256, H = 8, D = 32: 130 against 214 us).
    // EVO_FLAG_DEBUG_FWD_BIAS_TILES keeps the resident fp32 form, for comparison.
    return !p.bias || p.bias_dtype == p.dtype || (p.D == 8 && !p.gate) || (p.flags & EVO_FLAG_DEBUG_FWD_BIAS_TILES);
}

// The dK/dV kernel that walks over a chunk of S rows keeps 16-bit bias columns resident: it
// takes a bias in the dtype of q (or none) and rows whose length is a multiple of 8.  
// EVO_FLAG_DEBUG_NO_KV_RING selects the other kernel, for comparison.
static bool kv_ring_ok(const EvoAttnParams &p) {
    if ((p.flags & (EVO_FLAG_PER_PROBLEM | EVO_FLAG_DEBUG_NO_KV_RING)) || p.N <= 128 || p.N > mfma_kvr_max_n(p.D) || p.N % 8) return false;
    if (!aligned(p.lse, 16) || bias_direct(p)) return false;   // LSE rows are read four values at a time
    return !p.bias || p.bias_dtype == p.dtype;
}

// whether dQ of this call comes from the kernel over a chunk of rows in the form that also does the gate's pass
static bool gate_in_dq(const EvoAttnParams &p) {
    return mfma_ok(p, EVO_PASS_BWD) && !dq_split_ok(p) && !dq_wide_ok(p) && dq_ring_ok(p) && mfma_dqr_gate_ok(p.D, p.N);
}

static int launch_dq(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    if (dq_split_ok(p)) {
        EvoAttnParams q = p;
        q.dbias = nullptr;                       // dQ and delta first, then the dBias partials, which read delta
        if (const int rc = launch_mfma_dqw(q, e, st)) return rc;
        return launch_mfma_dbias(p, e, st);
    }
    if (dq_wide_ok(p)) return launch_mfma_dqw(p, e, st);
    return dq_ring_ok(p) ? launch_mfma_dqr(p, e, st) : launch_mfma_dq(p, e, st);
}

const char *evoattn_kernels(const EvoAttnParams *p, int pass) {
    if (!p) return "invalid";
    if (!mfma_ok(*p, pass)) return "generic";
    if (pass == EVO_PASS_FWD) return fwd_ring_ok(*p) ? "mfma_fwd_ring" : "mfma_fwd";
    const bool kvr = kv_ring_ok(*p);
    if (dq_split_ok(*p)) return kvr ? "mfma_dq_wide+mfma_dbias,mfma_dkdv_ring" : "mfma_dq_wide+mfma_dbias,mfma_dkdv";
    if (dq_wide_ok(*p)) return kvr ? "mfma_dq_wide,mfma_dkdv_ring" : "mfma_dq_wide,mfma_dkdv";
    if (kvr) return dq_ring_ok(*p) ? "mfma_dq_ring,mfma_dkdv_ring" : "mfma_dq,mfma_dkdv_ring";
    return dq_ring_ok(*p) ? "mfma_dq_ring,mfma_dkdv" : "mfma_dq,mfma_dkdv";
}

// the forward's launches for a checked parameter block whose `prep` is in place
static int fwd_launches(const EvoAttnParams &p, hipStream_t st) {
    Extra e{};
    e.vec_ok = bias_vec_ok(p);
    fill_prep(p, e);
    EVO_SET_TRACE(e);
    if (const int rc = launch_prep(p, e, st)) return rc;
    if (fwd_ring_ok(p)) return launch_mfma_fwdr(p, e, st);
    return launch_mfma_fwd(p, e, st);
}

int evoattn_fwd(const EvoAttnParams *p, void *hip_stream) {
    int rc = evoattn_check(p, EVO_PASS_FWD);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)hip_stream;
    if (!mfma_ok(*p, EVO_PASS_FWD)) return launch_generic_fwd(*p, st);
    if ((rc = check_prep(*p))) return rc;
    return fwd_launches(*p, st);
}

// Device address of this GPU's copy of `scratch`, asked for on the first call on that device.
static int static_prep(void **out) {
    static std::atomic<void *> addr[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return EVO_EHIP - (int)hipGetLastError();
    if (dev < 0 || dev >= 64) return EVO_EUNSUPPORTED;
    void *ptr = addr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !ptr) return EVO_EHIP - (int)(err != hipSuccess ? err : hipErrorInvalidSymbol);
        addr[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return EVO_OK;
}

int evoattn_fwd_static(const EvoAttnParams *p, void *hip_stream) {
    int rc = evoattn_check(p, EVO_PASS_FWD);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)hip_stream;
    if (!mfma_ok(*p, EVO_PASS_FWD)) return launch_generic_fwd(*p, st);   // those kernels take no prepared operands
    if (prep_layout(*p).total > (size_t)EVOATTN_STATIC_PREP_BYTES) return EVO_EWORKSPACE;
    EvoAttnParams q = *p;
    if ((rc = static_prep(&q.prep))) return rc;
    q.prep_bytes = (size_t)EVOATTN_STATIC_PREP_BYTES;
    // The prep kernel writes every byte of the array that this call's kernels read (bias tiles
    // with their zero tile, mask rows, flags), so nothing of an earlier call has to be cleared.
    return fwd_launches(q, st);
}

int evoattn_bwd(const EvoAttnParams *p0, void *hip_stream) {
    int rc = evoattn_check(p0, EVO_PASS_BWD);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)hip_stream;
    const WsLayout w = ws_layout(*p0);
    char *ws = (char *)p0->workspace;
    // With a gate, p0->dout is the gradient of the gated output: one pass over the rows forms the
    // gradient of the ungated output (into the workspace) and of the gate, and the attention
    // backward below runs on the former.
    EvoAttnParams ungated = *p0;
    Extra e{};
    if (p0->gate) {
        // (in place: a thread reads its 8 elements of dout before it writes them)
        void *d_o = (p0->flags & EVO_FLAG_GATE_DOUT_INPLACE) ? const_cast<void *>(p0->dout) : (void *)(ws + w.dout_ungated);
        ungated.dout = d_o;
        ungated.gate = nullptr;
        ungated.o_gated = nullptr;
        ungated.dgate = nullptr;
        // Where dQ comes from the kernel over a chunk of rows in its form for up to 256 keys at head dim 32, that
        // kernel does the gate's pass on the rows it stages anyway (it runs before the dK/dV kernel, which reads
        // the gradient of the ungated output it writes).
        if (gate_in_dq(ungated) && p0->o_gated && !(p0->flags & EVO_FLAG_ONLY_DKDV)) {
            e.gate_dout = p0->dout;
            e.gate_logits = p0->gate;
            e.gate_og = p0->o_gated;
            e.gate_dgate = p0->dgate;
        } else if ((rc = launch_gate_bwd(*p0, d_o, (float *)(ws + w.delta), st))) {
            return rc;
        }
    }
    const EvoAttnParams *p = &ungated;
    e.n_chunks = w.n_chunks;
    e.chunk = w.chunk;
    e.vec_ok = bias_vec_ok(*p);
    e.delta = (float *)(ws + w.delta);
    e.delta_given = p0->gate && !e.gate_dout ? 1 : 0;   // (the gate's pass wrote it; the dQ kernels then read no ungated O)
    e.shift = (float *)(ws + w.shift);
    e.dmask_part = (float *)(ws + w.dmask_part);
    e.dbias_part = (float *)(ws + w.dbias_part);
    if (!mfma_ok(*p, EVO_PASS_BWD)) return launch_generic_bwd(*p, e, st);
    if ((rc = check_prep(*p))) return rc;
    fill_prep(*p, e);
    EVO_SET_TRACE(e);
    if (!(p->flags & EVO_FLAG_PREP_VALID) && (rc = launch_prep(*p, e, st))) return rc;
    if (p->flags & EVO_FLAG_ONLY_DQ) return launch_dq(*p, e, st);
    const bool kvring = kv_ring_ok(*p);
    // that kernel sums the dBias partials on its way in (they lie 16-byte aligned for it)
    const bool partials = p->dbias && !dq_writes_dbias(*p);
    // (both dK/dV kernels do; the one-workgroup-per-problem kernel where the sums come in whole 16-byte pieces)
    const bool fused_reduce = partials && !(p->flags & EVO_FLAG_ONLY_DQ) && aligned(p->dbias, 16) &&
                              (kvring || ((int64_t)p->B * p->H * p->N * p->N) % 4 == 0);
    e.dbias_chunks = fused_reduce ? e.n_chunks : 0;
    if (p->flags & EVO_FLAG_ONLY_DKDV) return kvring ? launch_mfma_kvr(*p, e, st) : launch_mfma_dkdv(*p, e, st);
    // dQ first: it also writes delta, which the dK/dV kernel reads
    if ((rc = launch_dq(*p, e, st))) return rc;
    if ((rc = kvring ? launch_mfma_kvr(*p, e, st) : launch_mfma_dkdv(*p, e, st))) return rc;
    if (partials && !fused_reduce && (rc = launch_dbias_reduce(*p, e, st))) return rc;
    if (p->dmask && (rc = launch_dmask_reduce(*p, e, st))) return rc;
    return EVO_OK;
}

}  // extern "C"
