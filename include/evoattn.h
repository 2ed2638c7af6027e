/*
 * evoattn.h - C ABI of the MI355X (gfx950) Evoformer attention library.
 *
 * One attention "problem" is (b, h, s): N query rows against N key rows of width D,
 *     O = softmax(scale * Q K^T + pair_bias[b,h] + row_mask[b,s]) V.
 * The library holds the device kernels the reference generates with Triton; the host
 * (a torch.autograd.Function, a C++ trainer, ...) owns every buffer, hands in raw device
 * pointers, element strides and a HIP stream.  No entry point allocates, synchronises,
 * throws or touches any stream but the one it is given.  All return 0 or a negative
 * EVO_E* code; evoattn_strerror() names it.
 *
 * Reference interface each entry point stands in for (lvhoaa/evoformer_triton,
 * dsevoformer-triton/evoformer.py):
 *   evoattn_fwd  <- the `_attn_fwd[grid](...)` launch in EvoformerAttention.forward
 *                   (evoformer.py:676-724; kernels :23-297)
 *   evoattn_bwd  <- the three launches in EvoformerAttention.backward:
 *                   `_attn_bwd_preprocess` (:761-768), `_attn_bwd_dk_dv` (:776-812),
 *                   `_attn_bwd_dq` (:815-854), plus the zero-fill and the cast of
 *                   d_pair_bias (:752, :860)
 *   evoattn_prep_bytes, evoattn_bwd_workspace_bytes <- the `D = torch.empty_like(M)` and fp32 `d_pair_bias`
 *                   staging allocations (:752, :758), sized for the caller to make
 *   evoattn_check <- the asserts at :642-643 and :747-748
 */
#ifndef EVOATTN_H
#define EVOATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EVOATTN_VERSION 4   /* 2: gate, o_gated, dgate appended to EvoAttnParams; 3: LayerNorm and column-sum entry points,
                               EVO_FLAG_GATE_DOUT_INPLACE, a gate on a q-family with gaps (slots of a wider buffer);
                               4: with a gate `o` may be NULL (the gated output alone), the backward takes o_gated */

/* element types */
enum {
    EVO_NONE = -1,
    EVO_BF16 = 0,
    EVO_F16  = 1,
    EVO_F32  = 2   /* "check mode": every product and sum in fp32, no matrix cores */
};

/* row-mask encodings; mask is indexed [b][s][key], key contiguous */
enum {
    EVO_MASK_NONE = 0,
    EVO_MASK_BOOL = 1,  /* uint8, non-zero = keep; dropped keys score -FLT_MAX (evoformer.py:69) */
    EVO_MASK_F32  = 2,  /* additive */
    EVO_MASK_BF16 = 3,  /* additive */
    EVO_MASK_F16  = 4   /* additive */
};

/* flags */
enum {
    EVO_FLAG_FORCE_GENERIC = 1, /* run the plain fp32-arithmetic kernels whatever the dtype */
    EVO_FLAG_PREP_VALID    = 2, /* evoattn_bwd: `prep` still holds what evoattn_fwd wrote for the
                                   same bias and mask; skip re-deriving it */
    /* Measurement aids: enqueue a single phase of the matrix-core backward.  ONLY_DQ runs
     * the dQ kernel (dq, delta and the dBias partials, no final dBias sum); ONLY_DKDV runs
     * the dK/dV kernel and needs the delta a previous full call left in the same workspace. */
    EVO_FLAG_ONLY_DQ       = 4,
    EVO_FLAG_ONLY_DKDV     = 8,
    /* Measurement aid: run the one-workgroup-per-(b,h,s) forms of the forward and dQ kernels
     * also where the forms that walk over a chunk of S rows apply (same results). */
    EVO_FLAG_PER_PROBLEM   = 16,
    /* evoattn_bwd with a gate: the gradient of the ungated output, dout * sigmoid(g), overwrites `dout`
     * instead of going to the workspace, which then does not grow by q's extent.  For a caller that owns
     * the memory of `dout` and does not need it afterwards; not together with EVO_FLAG_ONLY_DQ / _ONLY_DKDV. */
    EVO_FLAG_GATE_DOUT_INPLACE = 0x80,
    /* Debug switches for A/B comparisons of kernel forms (same results, other kernels); a
     * production caller leaves them clear.  All other bits of `flags` must be zero. */
    EVO_FLAG_DEBUG_OTHER_WIDTH  = 0x100,  /* one-workgroup-per-problem kernels: the other of their two workgroup widths (4 / 8 waves) */
    EVO_FLAG_DEBUG_NO_KV_RING   = 0x200,  /* dK/dV: the one-workgroup-per-problem kernel instead of the chunk-of-rows one */
    EVO_FLAG_DEBUG_FWD_BIAS_TILES = 0x400, /* chunk-of-rows forward: prepared bias tiles as C operands instead of the caller's 16-bit rows */
    EVO_FLAG_DEBUG_BIAS_TILES   = 0x800,  /* S <= 4: prepare the bias tiles instead of reading the caller's bias */
    EVO_FLAG_DEBUG_NO_DQ_WIDE   = 0x1000, /* dQ: the kernels that split a row's keys over the waves, also without a dBias sum */
    EVO_FLAG_DEBUG_NO_DQ_SPLIT  = 0x2000  /* dQ + dBias in one kernel, also where dQ and the dBias partials come from two */
};
#define EVO_FLAG_ALL (1 | 2 | 4 | 8 | 16 | 0x80 | 0x100 | 0x200 | 0x400 | 0x800 | 0x1000 | 0x2000)

/* A problem (b, s) whose every key carries a mask value below this is a "dead row"; see lse below.
 * (An fp32 sum of such a mask value and a score of order one is the mask value: half a unit in the
 * last place of 5e8 is 16.) */
#define EVOATTN_SHIFT_THRESHOLD (-5.0e8f)

/* error codes */
enum {
    EVO_OK            = 0,
    EVO_EINVAL        = -1,  /* null pointer, non-positive size, bad enum */
    EVO_EUNSUPPORTED  = -2,  /* head dim or size outside what the kernels cover */
    EVO_EALIGN        = -3,  /* pointer or stride not aligned for the requested dtype */
    EVO_EWORKSPACE    = -4,  /* workspace missing or too small */
    EVO_EOVERFLOW     = -5,  /* extents overflow the index type */
    EVO_EHIP          = -100 /* EVO_EHIP - hipError_t from a launch */
};

enum { EVO_PASS_FWD = 0, EVO_PASS_BWD = 1 };

/*
 * Strides are in elements.  q, k, v, o, dout, dq, dk, dv all share one stride set:
 * element (b,h,s,n,d) lives at b*stride_b + h*stride_h + s*stride_s + n*stride_n + d.
 * The reference's flat reinterpretation of a dense [B,S,N,H,D] tensor as [B,H,S,N,D]
 * (evoformer.py:648-650) is (S*N*H*D, S*N*D, N*D, D); a true per-head view of the same
 * tensor is (S*N*H*D, D, N*H*D, H*D).
 * lse is dense [B][H][S][N] fp32.  For a problem whose every key carries a mask value
 * below EVOATTN_SHIFT_THRESHOLD (-5e8: the reference's fill for a bool mask, an additive
 * mask of -1e9) the scores are the mask values alone, less the largest of them (in the
 * reference's fp32 arithmetic q.k and the bias vanish next to such a mask: equal mask
 * values give uniform probabilities; the shift cancels in O and in every gradient), and
 * lse holds the log-sum-exp of those shifted scores.  A row masked throughout by less
 * (say -2e5) keeps q.k and the bias, rounded to the mask's last place as fp32 eager
 * rounds them (there the two agree as far as that rounding lets them: 1.6e-2 in a score
 * at -2e5).  Otherwise
 * lse = log sum_j exp(score_ij).
 */
typedef struct EvoAttnParams {
    int32_t B, S, N, H, D;
    int32_t dtype;        /* EVO_BF16 / EVO_F16 / EVO_F32 : q,k,v,o,dout,dq,dk,dv */
    int32_t bias_dtype;   /* EVO_NONE, EVO_F32, or equal to dtype */
    int32_t mask_kind;    /* EVO_MASK_* */
    int32_t dbias_dtype;  /* dtype of dbias: EVO_F32 or equal to dtype (ignored if dbias NULL) */
    int32_t flags;        /* EVO_FLAG_* */
    float   scale;        /* softmax scale, normally D^-0.5 (evoformer.py:646) */
    int32_t reserved;

    int64_t stride_b, stride_h, stride_s, stride_n;          /* q-family */
    int64_t bias_stride_b, bias_stride_h, bias_stride_row;    /* bias[b][h][row][col], col contiguous */
    int64_t mask_stride_b, mask_stride_s;                     /* mask[b][s][key], key contiguous */

    const void *q, *k, *v;
    const void *bias;     /* may be NULL (bias_dtype = EVO_NONE) */
    const void *mask;     /* may be NULL (mask_kind = EVO_MASK_NONE) */
    void       *o;        /* fwd: out; bwd: in (may be NULL with a gate, see below) */
    float      *lse;      /* fwd: out; bwd: in */

    const void *dout;     /* bwd only below */
    void       *dq, *dk, *dv;
    void       *dbias;    /* dense [B][H][N][N], may be NULL */
    float      *dmask;    /* dense [B][S][N] fp32 gradient of an additive mask, may be NULL */
    void       *workspace;
    size_t      workspace_bytes;

    /* Prepared operands (bias in accumulator-tile order, mask rows in log2 units): scratch
     * the matrix-core kernels derive from bias and mask at the start of evoattn_fwd.  The
     * caller provides evoattn_prep_bytes() bytes, 256-byte aligned; it may hand the same
     * buffer to evoattn_bwd with EVO_FLAG_PREP_VALID to skip the second derivation. */
    void       *prep;
    size_t      prep_bytes;

    /* Output gate of the Evoformer block, fused (all three NULL: no gate).  `gate` holds the gate
     * logits g, element for element like q (same dtype, same four strides).  evoattn_fwd then
     * writes Og = sigmoid(g) * O to o_gated (laid out like o) from its epilogue; the ungated O goes
     * to `o` as well if `o` is not NULL, and is not written at all if it is.  evoattn_bwd takes in
     * `dout` the gradient of Og and in `o_gated` the forward's Og (or, with o_gated NULL, the
     * ungated O in `o`), forms dO = dout * sigmoid(g), dgate = dout * Og * (1 - sigmoid(g)) and
     * delta = rowsum(dO * Og / sigmoid(g)) (= rowsum(dO * O)) in one pass over the rows (dgate laid out like
     * q; dO goes to the workspace, laid out like q, which grows by q's extent in memory) and runs
     * the attention backward on that dO and that delta: no ungated O is read.  The q-family may be
     * dense or a slot of a buffer of up to 8 such tensors (Q, K, V and the gate as slices of one
     * projection's result: strides of [B][S][N][W][H][D]), not sparser; with a gate every tensor
     * laid out like q starts on a 16-byte boundary and the four strides are multiples of 16 bytes
     * (else EVO_EALIGN: the gate's kernels move rows in 16-byte pieces), and H is at most 256.  The reference returns O
     * ungated (evoformer.py:735); its callers apply the gate as a separate step. */
    const void *gate;
    void       *o_gated;
    void       *dgate;
} EvoAttnParams;

int         evoattn_version(void);
const char *evoattn_strerror(int code);

/* Host-only validation of a parameter block for one pass; launches nothing. */
int evoattn_check(const EvoAttnParams *p, int pass);

/* Bytes of the `prep` buffer evoattn_fwd and evoattn_bwd need (0 on invalid input). */
size_t evoattn_prep_bytes(const EvoAttnParams *p);

/* Bytes of device workspace evoattn_bwd needs for this problem (0 on invalid input). */
size_t evoattn_bwd_workspace_bytes(const EvoAttnParams *p);

/* Enqueue the forward: writes o and lse. */
int evoattn_fwd(const EvoAttnParams *p, void *hip_stream);

/* evoattn_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose
 * forward allocates what it needs with torch (evoformer.py:654, 669-671).  Same kernels and results
 * as evoattn_fwd, but the prepared operands live in an array inside the library instead of the
 * caller's `prep` buffer: `prep` and `prep_bytes` of the parameter block are ignored, o and lse are
 * still the caller's, and the call makes no hipMalloc / hipFree and no allocating library call.
 * Limit: problems whose evoattn_prep_bytes() exceeds EVOATTN_STATIC_PREP_BYTES (16 MiB: rows up to
 * about 512 keys with 8 heads, e.g. B=1 S=512 N=256 H=8 needs 6.0 MB) return EVO_EWORKSPACE.  The
 * array is shared by every call on one GPU (each GPU has its own copy) and keeps the last call's
 * contents: calls that overlap in time on one GPU race on it, so enqueue them on one stream or
 * order them otherwise.  evoattn_bwd cannot reuse this prep (EVO_FLAG_PREP_VALID does not apply). */
#define EVOATTN_STATIC_PREP_BYTES (16u << 20)
int evoattn_fwd_static(const EvoAttnParams *p, void *hip_stream);

/* Enqueue the backward: writes dq, dk, dv and, when non-NULL, dbias and dmask.
 * Deterministic: no floating-point atomics; two runs give bit-identical results. */
int evoattn_bwd(const EvoAttnParams *p, void *hip_stream);

/* Name of the kernel family evoattn_fwd/evoattn_bwd would run for these parameters
 * ("mfma" or "generic"); for tests and reports. */
const char *evoattn_path(const EvoAttnParams *p, int pass);

/* Names of the main kernels that pass would launch, comma separated (e.g. "mfma_fwd_ring",
 * "mfma_dq_ring,mfma_dkdv", "mfma_dq_wide,mfma_dkdv", "generic"); for reports and profiles. */
const char *evoattn_kernels(const EvoAttnParams *p, int pass);

/* ---- LayerNorm of the block around the attention -------------------------------------------
 * No counterpart in the reference's operator, which starts at Q, K, V (evoformer.py:640-651): in
 * an Evoformer block the representation is normalised before the Q, K, V and gate projections and
 * the pair representation before the bias projection; these entry points do that normalisation
 * (over the last dimension of a dense [rows, cols] array) at the rate of HBM.
 *   dtype  EVO_BF16 / EVO_F16 / EVO_F32: x, y, gamma, beta, dy, dx, dgamma, dbeta
 *   cols   a multiple of 16 bytes' worth of elements, at most 2048 (1024 for fp32)
 *   gamma, beta, dx, dgamma, dbeta may be NULL (weight 1, bias 0; gradient not wanted)
 *   mean, rstd  [rows] fp32: written by the forward, read by the backward
 * All pointers 16-byte aligned.  The backward sums the gradients of gamma and beta through
 * `workspace` (evoattn_layernorm_bwd_workspace_bytes) in a fixed order: bit-reproducible.
 * Nothing is allocated or synchronised; everything runs on `hip_stream`. */
int evoattn_layernorm_fwd(const void *x, const void *gamma, const void *beta, void *y, float *mean, float *rstd,
                          int64_t rows, int32_t cols, int32_t dtype, float eps, void *hip_stream);
size_t evoattn_layernorm_bwd_workspace_bytes(int64_t rows, int32_t cols, int32_t dtype);
int evoattn_layernorm_bwd(const void *dy, const void *x, const void *gamma, const float *mean, const float *rstd,
                          void *dx, void *dgamma, void *dbeta, void *workspace, size_t workspace_bytes,
                          int64_t rows, int32_t cols, int32_t dtype, void *hip_stream);

/* Column sums of a [rows, cols] array whose rows lie `row_stride` elements apart (cols for a dense array;
 * more for some columns of a wider one), out[c] = sum over rows of a[r][c], in the dtype of a (fp32 sums
 * in a fixed order).  No counterpart in the reference's operator: the bias gradient of the block's
 * Linear layers (gate and output projection), one pass over the array at the rate of HBM.  Same limits
 * on cols and alignment as the LayerNorm entry points; `workspace` of evoattn_colsum_workspace_bytes(). */
size_t evoattn_colsum_workspace_bytes(int64_t rows, int32_t cols, int32_t dtype);
int evoattn_colsum(const void *a, int64_t row_stride, void *out, void *workspace, size_t workspace_bytes, int64_t rows,
                   int32_t cols, int32_t dtype, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* EVOATTN_H */
