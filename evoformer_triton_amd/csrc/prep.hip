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

__global__ void __launch_bounds__(256) prep_kernel(EvoAttnParams p, Extra e, unsigned n_bias_blocks) {
    __shared__ float red[4];
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
        const int kt = t % NT, qt = (t / NT) % NT;
        const int h = (t / NT / NT) % p.H, bb = t / NT / NT / p.H;
        const int li = lane & 31, g = lane >> 5, rr = tid >> 6;
        const int64_t base = (int64_t)bb * p.bias_stride_b + (int64_t)h * p.bias_stride_h;
        const int64_t o = ((int64_t)t * 64 + lane) * 16 + 4 * rr;
        if (e.bq16) {
            // the entries as given (the bias has the dtype of q: 16 bits, exact)
            const unsigned short *src = (const unsigned short *)p.bias + base;
            unsigned wq[4], wk[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int a = 8 * rr + 4 * g + i;  // accumulator row held by register 4rr+i
                const int q1 = qt * 32 + li, key1 = kt * 32 + a, q2 = qt * 32 + a, key2 = kt * 32 + li;
                wq[i] = (q1 < p.N && key1 < p.N) ? src[(int64_t)q1 * p.bias_stride_row + key1] : 0u;
                wk[i] = (q2 < p.N && key2 < p.N) ? src[(int64_t)q2 * p.bias_stride_row + key2] : 0u;
            }
            *reinterpret_cast<uint2 *>(e.bq16 + o) = make_uint2(wq[0] | (wq[1] << 16), wq[2] | (wq[3] << 16));
            *reinterpret_cast<uint2 *>(e.bk16 + o) = make_uint2(wk[0] | (wk[1] << 16), wk[2] | (wk[3] << 16));
        } else {
            f32x4 vq, vk;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int a = 8 * rr + 4 * g + i;
                {
                    const int q = qt * 32 + li, key = kt * 32 + a;
                    vq[i] = (q < p.N && key < p.N) ? kLog2e * bias_at(p, base + (int64_t)q * p.bias_stride_row + key) : 0.0f;
                }
                {
                    const int q = qt * 32 + a, key = kt * 32 + li;
                    vk[i] = (q < p.N && key < p.N) ? kLog2e * bias_at(p, base + (int64_t)q * p.bias_stride_row + key) : 0.0f;
                }
            }
            *reinterpret_cast<f32x4 *>(e.bq + o) = vq;
            *reinterpret_cast<f32x4 *>(e.bk + o) = vk;
        }
        if (e.bt) {
            // the same four entries of column `key` as given (the dtypes agree, so exact),
            // key-major: N is a multiple of 8 here, so the four are inside the matrix or not
            const int q = qt * 32 + 8 * rr + 4 * g, key = kt * 32 + li;
            if (q < p.N && key < p.N) {
                const int64_t src = base + (int64_t)q * p.bias_stride_row + key;
                const int64_t dst = (((int64_t)bb * p.H + h) * p.N + key) * p.N + q;
                unsigned short w[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) w[i] = ((const unsigned short *)p.bias)[src + (int64_t)i * p.bias_stride_row];
                *reinterpret_cast<uint2 *>((unsigned short *)e.bt + dst) =
                    make_uint2(w[0] | ((unsigned)w[1] << 16), w[2] | ((unsigned)w[3] << 16));
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
    const unsigned nb = p.bias && !e.bias_direct ? (unsigned)e.bias_batches * p.H * NT * NT + 1u : 0u;
    const unsigned nm = (unsigned)(p.B * p.S);
    prep_kernel<<<nb + nm, 256, 0, st>>>(p, e, nb);
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

}  // namespace evo
