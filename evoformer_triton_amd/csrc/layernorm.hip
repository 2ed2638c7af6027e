// LayerNorm over the last dimension, forward and backward, for the block around the attention
// (the normalisation of the representation before the Q, K, V and gate projections and of the
// pair representation before the bias projection).  The reference's operator starts at Q, K, V
// (evoformer.py:640-651); the model code around it normalises with the framework's LayerNorm.
//
// The work is bound by HBM: the forward reads x and writes y once, the backward reads x and dy
// and writes dx once.  A row is held in registers by a group of lanes (16 bytes per lane and
// piece, one to four pieces per lane), so mean, variance and the two sums of the backward are
// register sums followed by a few cross-lane steps; a workgroup walks over rows with a grid
// stride.  The gradients of weight and bias are summed per lane over the rows a workgroup
// visits, then over the workgroup in LDS, written as one partial per workgroup and added up
// by a second small kernel in a fixed order: no atomics, bit-reproducible.
#include "common.h"
#include "bwd_common.h"

namespace evo {

constexpr int kLnThreads = 256;
constexpr int kLnMaxPieces = 4;       // 16-byte pieces of a row per lane
constexpr int kLnFwdBlocks = 4096;    // most workgroups of the forward
constexpr int kLnBwdBlocks = 1024;    // most workgroups of the backward = partial sums of the weight and bias gradients

template <typename T>
struct LnVec {
    static constexpr int N = 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
};

// how a row is spread over lanes: `lpr` lanes (a power of two, at most 64), `pieces` 16-byte pieces per lane
struct LnShape {
    int lpr, pieces;
};

static LnShape ln_shape(int cols, int vec) {
    const int n = cols / vec;          // 16-byte pieces per row
    int lpr = 1;
    while (lpr < 64 && lpr < n) lpr *= 2;
    return {lpr, (n + lpr - 1) / lpr};
}

__device__ __forceinline__ float ln_group_sum(float s, int lpr) {
    for (int o = lpr >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
    return s;
}

template <typename T, int PIECES>
__global__ void __launch_bounds__(kLnThreads)
ln_fwd_kernel(const T *__restrict__ x, const T *__restrict__ gamma, const T *__restrict__ beta, T *__restrict__ y,
              float *__restrict__ mean, float *__restrict__ rstd, int64_t rows, int cols, float eps, int lpr) {
    constexpr int VEC = LnVec<T>::N;
    typedef typename LnVec<T>::type vT;
    const int tid = threadIdx.x, sub = tid % lpr, grp = tid / lpr, rpb = kLnThreads / lpr;
    const int npieces = cols / VEC;
    float g[PIECES][VEC], b[PIECES][VEC];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int pc = i * lpr + sub;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            g[i][e] = 1.0f;
            b[i][e] = 0.0f;
        }
        if (pc < npieces) {
            if (gamma) {
                const vT w = *reinterpret_cast<const vT *>(gamma + pc * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) g[i][e] = (float)w[e];
            }
            if (beta) {
                const vT w = *reinterpret_cast<const vT *>(beta + pc * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) b[i][e] = (float)w[e];
            }
        }
    }
    const float inv = 1.0f / (float)cols;
    for (int64_t row = (int64_t)blockIdx.x * rpb + grp; row < rows; row += (int64_t)gridDim.x * rpb) {
        float v[PIECES][VEC];
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int pc = i * lpr + sub;
            if (pc < npieces) {
                const vT raw = *reinterpret_cast<const vT *>(x + row * cols + pc * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    v[i][e] = (float)raw[e];
                    s += v[i][e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) v[i][e] = 0.0f;
            }
        }
        const float mu = ln_group_sum(s, lpr) * inv;
        float q = 0.0f;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            if (i * lpr + sub < npieces) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float d = v[i][e] - mu;
                    q += d * d;
                }
            }
        }
        const float r = 1.0f / sqrtf(ln_group_sum(q, lpr) * inv + eps);
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int pc = i * lpr + sub;
            if (pc < npieces) {
                vT out;
#pragma unroll
                for (int e = 0; e < VEC; ++e) out[e] = (T)((v[i][e] - mu) * r * g[i][e] + b[i][e]);
                *reinterpret_cast<vT *>(y + row * cols + pc * VEC) = out;
            }
        }
        if (sub == 0) {
            mean[row] = mu;
            rstd[row] = r;
        }
    }
}

// part: [gridDim.x][2][cols] fp32, the workgroup's sums of dy * xhat (weight) and of dy (bias)
template <typename T, int PIECES>
__global__ void __launch_bounds__(kLnThreads)
ln_bwd_kernel(const T *__restrict__ dy, const T *__restrict__ x, const T *__restrict__ gamma, const float *__restrict__ mean,
              const float *__restrict__ rstd, T *__restrict__ dx, float *__restrict__ part, int64_t rows, int cols, int lpr) {
    constexpr int VEC = LnVec<T>::N;
    typedef typename LnVec<T>::type vT;
    __shared__ float red[kLnThreads * PIECES * VEC];      // [rows per workgroup][lpr * PIECES * VEC]
    const int tid = threadIdx.x, sub = tid % lpr, grp = tid / lpr, rpb = kLnThreads / lpr;
    const int npieces = cols / VEC;
    float g[PIECES][VEC], dg[PIECES][VEC], db[PIECES][VEC];
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
        const int pc = i * lpr + sub;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            g[i][e] = 1.0f;
            dg[i][e] = 0.0f;
            db[i][e] = 0.0f;
        }
        if (gamma && pc < npieces) {
            const vT w = *reinterpret_cast<const vT *>(gamma + pc * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) g[i][e] = (float)w[e];
        }
    }
    const float inv = 1.0f / (float)cols;
    for (int64_t row = (int64_t)blockIdx.x * rpb + grp; row < rows; row += (int64_t)gridDim.x * rpb) {
        const float mu = mean[row], r = rstd[row];
        float xh[PIECES][VEC], gy[PIECES][VEC];
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int pc = i * lpr + sub;
            if (pc < npieces) {
                const vT xr = *reinterpret_cast<const vT *>(x + row * cols + pc * VEC);
                const vT dr = *reinterpret_cast<const vT *>(dy + row * cols + pc * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float d = (float)dr[e];
                    xh[i][e] = ((float)xr[e] - mu) * r;
                    gy[i][e] = d * g[i][e];
                    s1 += gy[i][e];
                    s2 += gy[i][e] * xh[i][e];
                    dg[i][e] += d * xh[i][e];
                    db[i][e] += d;
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) xh[i][e] = gy[i][e] = 0.0f;
            }
        }
        if (dx) {   // uniform
            const float c1 = ln_group_sum(s1, lpr) * inv, c2 = ln_group_sum(s2, lpr) * inv;
#pragma unroll
            for (int i = 0; i < PIECES; ++i) {
                const int pc = i * lpr + sub;
                if (pc < npieces) {
                    vT out;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) out[e] = (T)((gy[i][e] - c1 - xh[i][e] * c2) * r);
                    *reinterpret_cast<vT *>(dx + row * cols + pc * VEC) = out;
                }
            }
        }
    }
    if (!part) return;   // uniform
    // the workgroup's sums: the row groups meet in LDS, first for the weight, then for the bias
    const int pitch = lpr * PIECES * VEC;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int i = 0; i < PIECES; ++i)
#pragma unroll
            for (int e = 0; e < VEC; ++e) red[grp * pitch + (i * lpr + sub) * VEC + e] = pass == 0 ? dg[i][e] : db[i][e];
        __syncthreads();
        for (int c = tid; c < cols; c += kLnThreads) {
            float s = 0.0f;
            for (int r2 = 0; r2 < rpb; ++r2) s += red[r2 * pitch + c];
            part[((int64_t)blockIdx.x * 2 + pass) * cols + c] = s;
        }
        __syncthreads();
    }
}

// Column sums of a dense [rows, cols] array (the bias gradient of a Linear layer): the same walk over
// the rows as the LayerNorm backward, one partial [cols] per workgroup.
template <typename T, int PIECES>
__global__ void __launch_bounds__(kLnThreads)
colsum_kernel(const T *__restrict__ a, float *__restrict__ part, int64_t rows, int cols, int64_t row_stride, int lpr) {
    constexpr int VEC = LnVec<T>::N;
    typedef typename LnVec<T>::type vT;
    __shared__ float red[kLnThreads * PIECES * VEC];
    const int tid = threadIdx.x, sub = tid % lpr, grp = tid / lpr, rpb = kLnThreads / lpr;
    const int npieces = cols / VEC;
    float acc[PIECES][VEC];
#pragma unroll
    for (int i = 0; i < PIECES; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[i][e] = 0.0f;
    for (int64_t row = (int64_t)blockIdx.x * rpb + grp; row < rows; row += (int64_t)gridDim.x * rpb) {
#pragma unroll
        for (int i = 0; i < PIECES; ++i) {
            const int pc = i * lpr + sub;
            if (pc < npieces) {
                const vT v = *reinterpret_cast<const vT *>(a + row * row_stride + pc * VEC);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[i][e] += (float)v[e];
            }
        }
    }
    const int pitch = lpr * PIECES * VEC;
#pragma unroll
    for (int i = 0; i < PIECES; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[grp * pitch + (i * lpr + sub) * VEC + e] = acc[i][e];
    __syncthreads();
    for (int c = tid; c < cols; c += kLnThreads) {
        float s = 0.0f;
        for (int r2 = 0; r2 < rpb; ++r2) s += red[r2 * pitch + c];
        part[(int64_t)blockIdx.x * cols + c] = s;
    }
}

// dgamma, dbeta = the sums of the partials over the workgroups, in a fixed order (`narr` arrays per partial:
// two for the LayerNorm backward, one for plain column sums, whose result goes to `dgamma`).  A workgroup takes 4
// columns and splits the partials over 64 threads per column, four rows in flight per thread (one
// thread per column walking over a thousand partials waits for a thousand loads in turn: 64 us).
constexpr int kLnRedCols = 4, kLnRedSlices = 64;
template <typename T>
__global__ void __launch_bounds__(kLnRedCols * kLnRedSlices)
ln_reduce_kernel(const float *__restrict__ part, int nblk, int narr, int cols, T *__restrict__ dgamma, T *__restrict__ dbeta) {
    __shared__ float red[2][kLnRedCols][kLnRedSlices];
    const int cq = threadIdx.x % kLnRedCols, rs = threadIdx.x / kLnRedCols, c = blockIdx.x * kLnRedCols + cq;
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f}, b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (c < cols) {
        int k = rs;
        for (; k + 3 * kLnRedSlices < nblk; k += 4 * kLnRedSlices) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float *row = part + (int64_t)(k + u * kLnRedSlices) * narr * cols;
                a[u] += row[c];
                if (narr == 2) b[u] += row[cols + c];
            }
        }
        for (; k < nblk; k += kLnRedSlices) {
            const float *row = part + (int64_t)k * narr * cols;
            a[0] += row[c];
            if (narr == 2) b[0] += row[cols + c];
        }
    }
    red[0][cq][rs] = (a[0] + a[1]) + (a[2] + a[3]);
    red[1][cq][rs] = (b[0] + b[1]) + (b[2] + b[3]);
    __syncthreads();
    if (threadIdx.x < 2 * kLnRedCols) {
        const int which = threadIdx.x / kLnRedCols, col = blockIdx.x * kLnRedCols + threadIdx.x % kLnRedCols;
        float s = 0.0f;
        for (int i = 0; i < kLnRedSlices; ++i) s += red[which][threadIdx.x % kLnRedCols][i];
        T *out = which == 0 ? dgamma : dbeta;
        if (col < cols && out) out[col] = (T)s;
    }
}

static int ln_elem_bytes(int dtype) { return dtype == EVO_F32 ? 4 : (dtype == EVO_BF16 || dtype == EVO_F16) ? 2 : 0; }

static int ln_check(int64_t rows, int cols, int dtype) {
    const int eb = ln_elem_bytes(dtype);
    if (!eb || rows < 0 || cols <= 0) return EVO_EINVAL;
    const int vec = 16 / eb;
    if (cols % vec) return EVO_EALIGN;
    if (cols / vec > 64 * kLnMaxPieces) return EVO_EUNSUPPORTED;
    if (rows > ((int64_t)1 << 40)) return EVO_EOVERFLOW;
    return EVO_OK;
}

static bool ln_misaligned(const void *p) { return p && ((uintptr_t)p & 15) != 0; }

static unsigned ln_blocks(int64_t rows, int lpr, int most) {
    const int64_t rpb = kLnThreads / lpr, want = (rows + rpb - 1) / rpb;
    return (unsigned)(want < most ? want : most);
}

template <typename T>
static int ln_fwd_launch(const void *x, const void *gamma, const void *beta, void *y, float *mean, float *rstd, int64_t rows,
                         int cols, float eps, hipStream_t st) {
    const LnShape s = ln_shape(cols, LnVec<T>::N);
    const unsigned grid = ln_blocks(rows, s.lpr, kLnFwdBlocks);
    auto go = [&](auto kern) {
        kern<<<grid, kLnThreads, 0, st>>>((const T *)x, (const T *)gamma, (const T *)beta, (T *)y, mean, rstd, rows, cols, eps, s.lpr);
    };
    if (s.pieces == 1) go(ln_fwd_kernel<T, 1>);
    else if (s.pieces == 2) go(ln_fwd_kernel<T, 2>);
    else go(ln_fwd_kernel<T, 4>);
    return hip_rc();
}

template <typename T>
static int ln_bwd_launch(const void *dy, const void *x, const void *gamma, const float *mean, const float *rstd, void *dx,
                         void *dgamma, void *dbeta, float *part, int64_t rows, int cols, hipStream_t st) {
    const LnShape s = ln_shape(cols, LnVec<T>::N);
    const unsigned grid = ln_blocks(rows, s.lpr, kLnBwdBlocks);
    const bool sums = dgamma || dbeta;
    auto go = [&](auto kern) {
        kern<<<grid, kLnThreads, 0, st>>>((const T *)dy, (const T *)x, (const T *)gamma, mean, rstd, (T *)dx, sums ? part : nullptr,
                                          rows, cols, s.lpr);
    };
    if (rows > 0) {
        if (s.pieces == 1) go(ln_bwd_kernel<T, 1>);
        else if (s.pieces == 2) go(ln_bwd_kernel<T, 2>);
        else go(ln_bwd_kernel<T, 4>);
        if (const int rc = hip_rc()) return rc;
    }
    if (sums) {   // (no rows: no partials, the sums are zero)
        ln_reduce_kernel<T><<<(cols + kLnRedCols - 1) / kLnRedCols, kLnRedCols * kLnRedSlices, 0, st>>>(part, rows > 0 ? (int)grid : 0, 2, cols, (T *)dgamma, (T *)dbeta);
        return hip_rc();
    }
    return EVO_OK;
}

template <typename T>
static int colsum_launch(const void *a, void *out, float *part, int64_t rows, int cols, int64_t row_stride, hipStream_t st) {
    const LnShape s = ln_shape(cols, LnVec<T>::N);
    const unsigned grid = ln_blocks(rows, s.lpr, kLnBwdBlocks);
    auto go = [&](auto kern) { kern<<<grid, kLnThreads, 0, st>>>((const T *)a, part, rows, cols, row_stride, s.lpr); };
    if (rows > 0) {
        if (s.pieces == 1) go(colsum_kernel<T, 1>);
        else if (s.pieces == 2) go(colsum_kernel<T, 2>);
        else go(colsum_kernel<T, 4>);
        if (const int rc = hip_rc()) return rc;
    }
    ln_reduce_kernel<T><<<(cols + kLnRedCols - 1) / kLnRedCols, kLnRedCols * kLnRedSlices, 0, st>>>(part, rows > 0 ? (int)grid : 0, 1, cols,
                                                                                                  (T *)out, (T *)nullptr);
    return hip_rc();
}

}  // namespace evo

extern "C" {

int evoattn_layernorm_fwd(const void *x, const void *gamma, const void *beta, void *y, float *mean, float *rstd, int64_t rows,
                          int32_t cols, int32_t dtype, float eps, void *hip_stream) {
    using namespace evo;
    if (const int rc = ln_check(rows, cols, dtype)) return rc;
    if (!x || !y || !mean || !rstd || !(eps >= 0.0f)) return EVO_EINVAL;
    if (ln_misaligned(x) || ln_misaligned(y) || ln_misaligned(gamma) || ln_misaligned(beta)) return EVO_EALIGN;
    if (rows == 0) return EVO_OK;
    hipStream_t st = (hipStream_t)hip_stream;
    switch (dtype) {
        case EVO_BF16: return ln_fwd_launch<bf16_t>(x, gamma, beta, y, mean, rstd, rows, cols, eps, st);
        case EVO_F16: return ln_fwd_launch<f16_t>(x, gamma, beta, y, mean, rstd, rows, cols, eps, st);
        default: return ln_fwd_launch<float>(x, gamma, beta, y, mean, rstd, rows, cols, eps, st);
    }
}

size_t evoattn_layernorm_bwd_workspace_bytes(int64_t rows, int32_t cols, int32_t dtype) {
    using namespace evo;
    if (ln_check(rows, cols, dtype) != EVO_OK) return 0;
    return (size_t)kLnBwdBlocks * 2 * (size_t)cols * sizeof(float);
}

int evoattn_layernorm_bwd(const void *dy, const void *x, const void *gamma, const float *mean, const float *rstd, void *dx,
                          void *dgamma, void *dbeta, void *workspace, size_t workspace_bytes, int64_t rows, int32_t cols,
                          int32_t dtype, void *hip_stream) {
    using namespace evo;
    if (const int rc = ln_check(rows, cols, dtype)) return rc;
    if (!dy || !x || !mean || !rstd || (!dx && !dgamma && !dbeta)) return EVO_EINVAL;
    if (ln_misaligned(dy) || ln_misaligned(x) || ln_misaligned(gamma) || ln_misaligned(dx)) return EVO_EALIGN;
    if ((dgamma || dbeta) && (!workspace || workspace_bytes < evoattn_layernorm_bwd_workspace_bytes(rows, cols, dtype)))
        return EVO_EWORKSPACE;
    if (ln_misaligned(workspace)) return EVO_EALIGN;
    hipStream_t st = (hipStream_t)hip_stream;
    float *part = (float *)workspace;
    switch (dtype) {
        case EVO_BF16: return ln_bwd_launch<bf16_t>(dy, x, gamma, mean, rstd, dx, dgamma, dbeta, part, rows, cols, st);
        case EVO_F16: return ln_bwd_launch<f16_t>(dy, x, gamma, mean, rstd, dx, dgamma, dbeta, part, rows, cols, st);
        default: return ln_bwd_launch<float>(dy, x, gamma, mean, rstd, dx, dgamma, dbeta, part, rows, cols, st);
    }
}

size_t evoattn_colsum_workspace_bytes(int64_t rows, int32_t cols, int32_t dtype) {
    using namespace evo;
    if (ln_check(rows, cols, dtype) != EVO_OK) return 0;
    return (size_t)kLnBwdBlocks * (size_t)cols * sizeof(float);
}

int evoattn_colsum(const void *a, int64_t row_stride, void *out, void *workspace, size_t workspace_bytes, int64_t rows, int32_t cols,
                   int32_t dtype, void *hip_stream) {
    using namespace evo;
    if (const int rc = ln_check(rows, cols, dtype)) return rc;
    if (!a || !out || row_stride < cols) return EVO_EINVAL;
    if (row_stride % (16 / ln_elem_bytes(dtype))) return EVO_EALIGN;
    if (ln_misaligned(a) || ln_misaligned(workspace)) return EVO_EALIGN;
    if (!workspace || workspace_bytes < evoattn_colsum_workspace_bytes(rows, cols, dtype)) return EVO_EWORKSPACE;
    hipStream_t st = (hipStream_t)hip_stream;
    float *part = (float *)workspace;
    switch (dtype) {
        case EVO_BF16: return colsum_launch<bf16_t>(a, out, part, rows, cols, row_stride, st);
        case EVO_F16: return colsum_launch<f16_t>(a, out, part, rows, cols, row_stride, st);
        default: return colsum_launch<float>(a, out, part, rows, cols, row_stride, st);
    }
}

}  // extern "C"
