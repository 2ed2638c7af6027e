// Operand preparation for the matrix-core kernels: one launch that rewrites the two small
// broadcast operands of the attention, the pair bias and the row mask, into the form the
// hot loops consume without any per-score arithmetic.
//
//  * bias -> two copies in 32x32 accumulator-tile order (64 lanes x 16 registers contiguous
//    per tile), one with lane = query (for S^T = K Q^T tiles) and one with lane = key (for
//    S = Q K^T tiles): the bias add of the reference (evoformer.py:68, :450, :594) becomes
//    the C operand of the score matmul.  An fp32 bias is stored as fp32 scaled by log2(e) and
//    a kernel loads a tile straight into the MFMA accumulator; a bias in the dtype of q is
//    stored as given, 16 bits per entry: the kernels read half the bytes and multiply by
//    log2(e) themselves, in fp32 (the same product).
//  * mask -> one row per (b, s), in log2 units, clamped to a finite floor, padded to a
//    multiple of 32 keys with the floor, each value already split into three 16-bit terms
//    (hi + mid + lo, exact to 24 bits) of the q/k/v element type.  The kernels carry them as
//    extra columns of K against ones in Q, so the mask (evoformer.py:69) is added by the
//    score matmul as well.
//  * dead[b][s] = 1 where every key of the row is masked below the threshold.  The
//    reference's fp32 scores are then all equal (the fill value swamps q.k and the bias), the
//    softmax is uniform over the keys; the kernels reproduce that by zeroing Q and the bias
//    for the row and subtracting the largest mask value from the mask.
#include "common.h"
#include "kernels.h"

namespace evo {

__device__ __forceinline__ float bias_at(const EvoAttnParams &p, int64_t off) {
    if (p.bias_dtype == EVO_F32) return ((const float *)p.bias)[off];
    if (p.bias_dtype == EVO_BF16) return (float)((const bf16_t *)p.bias)[off];
    return (float)((const f16_t *)p.bias)[off];
}

// A workgroup rewrites a strip of 32 query rows x kPrepStrip key tiles: the strip is read once, with the lanes along
// the rows (256 contiguous bytes per row for a 16-bit bias, where a single 32 x 32 tile has 64), and every lane slot
// of the tiles (16 entries: 32 or 64 contiguous bytes) is written by one thread.  (One workgroup per tile, its threads
// gathering two-byte entries and storing 8-byte pieces, moved 1.5 TB/s: 136 us for the 8 x 2048^2 entries of a
// 16-bit bias.)
constexpr int kPrepStrip = 4;
constexpr int kPrepCols = kPrepStrip * 32;

__global__ void __launch_bounds__(256) prep_kernel(EvoAttnParams p, Extra e, unsigned n_bias_blocks) {
    __shared__ float red[4];
    __shared__ __attribute__((aligned(16))) unsigned char strip[32 * (kPrepCols * 4 + 16)];
    const int tid = threadIdx.x, lane = tid & 63;
    const int NT = (p.N + 31) / 32;
    if (blockIdx.x < n_bias_blocks) {
        const unsigned t = blockIdx.x;
        if (t == n_bias_blocks - 1) {  // the all-zero tile
            if (e.bq16) {
                *reinterpret_cast<uint2 *>(e.bq16 + e.zero_tile + tid * 4) = make_uint2(0u, 0u);
                *reinterpret_cast<uint2 *>(e.bk16 + e.zero_tile + tid * 4) = make_uint2(0u, 0u);
            } else {
                const f32x4 z = {0.f, 0.f, 0.f, 0.f};
                *reinterpret_cast<f32x4 *>(e.bq + e.zero_tile + tid * 4) = z;
                *reinterpret_cast<f32x4 *>(e.bk + e.zero_tile + tid * 4) = z;
            }
            return;
        }
        const int NS = (NT + kPrepStrip - 1) / kPrepStrip;
        const int kt0 = (t % NS) * kPrepStrip, qt = (t / NS) % NT;
        const int h = (t / NS / NT) % p.H, bb = t / NS / NT / p.H;
        const int ntile = min(kPrepStrip, NT - kt0);
        const int64_t base = (int64_t)bb * p.bias_stride_b + (int64_t)h * p.bias_stride_h;
        const int q0 = qt * 32, k0 = kt0 * 32;
        const int li = lane & 31, g = lane >> 5, tl = tid >> 6;
        const int64_t tile0 = (((int64_t)bb * p.H + h) * NT + qt) * NT + kt0;
        if (e.bq16) {
            // the entries as given (the bias has the dtype of q: 16 bits, exact)
            constexpr int PITCH = kPrepCols + 8;                       // entries; rows 16 bytes further apart than long
            unsigned short(*sm)[PITCH] = reinterpret_cast<unsigned short(*)[PITCH]>(strip);
            const unsigned short *src = (const unsigned short *)p.bias + base;
            const bool vec = p.N % 8 == 0 && ((uintptr_t)p.bias & 15) == 0 && p.bias_stride_b % 8 == 0 &&
                             p.bias_stride_h % 8 == 0 && p.bias_stride_row % 8 == 0;   // uniform
            for (int idx = tid; idx < 32 * (kPrepCols / 8); idx += 256) {
                const int r = idx / (kPrepCols / 8), c = (idx % (kPrepCols / 8)) * 8;
                const int q = q0 + r, key = k0 + c;
                uint4 v = make_uint4(0u, 0u, 0u, 0u);
                if (q < p.N && key < p.N) {
                    const unsigned short *s8 = src + (int64_t)q * p.bias_stride_row + key;
                    if (vec) {
                        v = *reinterpret_cast<const uint4 *>(s8);
                    } else {
                        unsigned short w[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i) w[i] = key + i < p.N ? s8[i] : (unsigned short)0;
                        v = make_uint4(w[0] | ((unsigned)w[1] << 16), w[2] | ((unsigned)w[3] << 16),
                                       w[4] | ((unsigned)w[5] << 16), w[6] | ((unsigned)w[7] << 16));
                    }
                }
                *reinterpret_cast<uint4 *>(&sm[r][c]) = v;
            }
            __syncthreads();
            if (tl < ntile) {
                // lane slot (tile tl, lane): register r holds accumulator row 8 (r / 4) + 4 g + r % 4
                unsigned short wq[16], wk[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int a = 8 * (r >> 2) + 4 * g + (r & 3);
                    wq[r] = sm[li][tl * 32 + a];     // lane = query, register = key
                    wk[r] = sm[a][tl * 32 + li];     // lane = key, register = query
                }
                const int64_t o = ((tile0 + tl) * 64 + lane) * 16;
                uint4 *dq = reinterpret_cast<uint4 *>(e.bq16 + o), *dk = reinterpret_cast<uint4 *>(e.bk16 + o);
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    dq[hh] = make_uint4(wq[8 * hh] | ((unsigned)wq[8 * hh + 1] << 16), wq[8 * hh + 2] | ((unsigned)wq[8 * hh + 3] << 16),
                                        wq[8 * hh + 4] | ((unsigned)wq[8 * hh + 5] << 16), wq[8 * hh + 6] | ((unsigned)wq[8 * hh + 7] << 16));
                    dk[hh] = make_uint4(wk[8 * hh] | ((unsigned)wk[8 * hh + 1] << 16), wk[8 * hh + 2] | ((unsigned)wk[8 * hh + 3] << 16),
                                        wk[8 * hh + 4] | ((unsigned)wk[8 * hh + 5] << 16), wk[8 * hh + 6] | ((unsigned)wk[8 * hh + 7] << 16));
                }
            }
            if (e.bt) {
                // the strip transposed (key-major), as given: eight queries of one key per 16-byte store (N is a
                // multiple of 8 here, so the eight are inside the matrix or not)
                for (int idx = tid; idx < kPrepCols * 4; idx += 256) {
                    const int c = idx >> 2, qg = (idx & 3) * 8;
                    const int key = k0 + c, q = q0 + qg;
                    if (key < p.N && q < p.N) {
                        unsigned short w[8];
#pragma unroll
                        for (int i = 0; i < 8; ++i) w[i] = sm[qg + i][c];
                        const int64_t dst = (((int64_t)bb * p.H + h) * p.N + key) * p.N + q;
                        *reinterpret_cast<uint4 *>((unsigned short *)e.bt + dst) =
                            make_uint4(w[0] | ((unsigned)w[1] << 16), w[2] | ((unsigned)w[3] << 16),
                                       w[4] | ((unsigned)w[5] << 16), w[6] | ((unsigned)w[7] << 16));
                    }
                }
            }
        } else {
            // fp32 tiles in log2 units
            constexpr int PITCH = kPrepCols + 4;
            float(*sm)[PITCH] = reinterpret_cast<float(*)[PITCH]>(strip);
            const bool vec = p.bias_dtype == EVO_F32 && p.N % 4 == 0 && ((uintptr_t)p.bias & 15) == 0 && p.bias_stride_b % 4 == 0 &&
                             p.bias_stride_h % 4 == 0 && p.bias_stride_row % 4 == 0;   // uniform
            for (int idx = tid; idx < 32 * (kPrepCols / 4); idx += 256) {
                const int r = idx / (kPrepCols / 4), c = (idx % (kPrepCols / 4)) * 4;
                const int q = q0 + r, key = k0 + c;
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (q < p.N && key < p.N) {
                    const int64_t off = base + (int64_t)q * p.bias_stride_row + key;
                    if (vec) {
                        v = *reinterpret_cast<const f32x4 *>((const float *)p.bias + off);
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) v[i] = key + i < p.N ? bias_at(p, off + i) : 0.0f;
                    }
                }
                *reinterpret_cast<f32x4 *>(&sm[r][c]) = v * kLog2e;
            }
            __syncthreads();
            if (tl < ntile) {
                const int64_t o = ((tile0 + tl) * 64 + lane) * 16;
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    f32x4 vq, vk;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int a = 8 * m + 4 * g + i;
                        vq[i] = sm[li][tl * 32 + a];
                        vk[i] = sm[a][tl * 32 + li];
                    }
                    *reinterpret_cast<f32x4 *>(e.bq + o + 4 * m) = vq;
                    *reinterpret_cast<f32x4 *>(e.bk + o + 4 * m) = vk;
                }
            }
        }
        return;
    }
    const unsigned row = blockIdx.x - n_bias_blocks;  // (b, s)
    const int b = row / p.S, s = row % p.S;
    const int npad = NT * 32;
    float mx = -INFINITY;
    for (int j = tid; j < p.N; j += 256) mx = fmaxf(mx, fmaxf(mask_add(p, b, s, j), kMaskFloor));
    mx = wave_max(mx);
    if (lane == 0) red[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const bool dead = p.mask_kind != EVO_MASK_NONE && mx < kShiftThreshold;
    uint2 *out = e.m2 + (int64_t)row * npad;
    for (int j = tid; j < npad; j += 256) {
        float v = kMaskFloor;
        if (j < p.N) {
            float m = fmaxf(mask_add(p, b, s, j), kMaskFloor);
            if (dead) m -= mx;
            v = fmaxf(m * kLog2e, kMaskFloor);
        }
        out[j] = p.dtype == EVO_F16 ? pack_split3<f16_t>(v) : pack_split3<bf16_t>(v);
    }
    const int np256 = (p.N + 255) / 256 * 256;
    uint4 *outa = e.m2a + (int64_t)row * np256;
    const uint2 fl = p.dtype == EVO_F16 ? pack_split3<f16_t>(kMaskFloor) : pack_split3<bf16_t>(kMaskFloor);
    // (hi, mid, lo, 1, 1, 1, 0, 0): the ones meet the -LSE columns of the backward's score
    // MFMA; the forward multiplies them by zeros
    const unsigned one = p.dtype == EVO_F16 ? 0x3C00u : 0x3F80u;
    for (int j = tid; j < np256; j += 256) {
        const uint2 v = j < npad ? out[j] : fl;
        outa[j] = make_uint4(v.x, v.y | (one << 16), one | (one << 16), 0u);
    }
    if (tid == 0) e.dead[row] = dead ? 1 : 0;
}

int launch_prep(const EvoAttnParams &p, const Extra &e, hipStream_t st) {
    const unsigned NT = (p.N + 31) / 32;
    // (no bias tiles where the kernels read the caller's tensor)
    const unsigned NS = (NT + kPrepStrip - 1) / kPrepStrip;
    const unsigned nb = p.bias && !e.bias_direct ? (unsigned)e.bias_batches * p.H * NT * NS + 1u : 0u;
    const unsigned nm = (unsigned)(p.B * p.S);
    prep_kernel<<<nb + nm, 256, 0, st>>>(p, e, nb);
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

}  // namespace evo
