// Pieces shared by the backward matrix-core kernels of one head dim.
#pragma once

#include <atomic>

#include "common.h"

namespace evo {

// Geometry shared by the two kernels for head dim D.
template <int D>
struct Geo {
    static constexpr bool AUG_IN_PAD = D == 8;           // extra columns fit the zero padding of k-step 0
    static constexpr int KW = AUG_IN_PAD ? 16 : D + 16;  // operand row: data, extra columns, zeros
    static constexpr int KS = KW / 16;
    static constexpr int KSD = (D + 15) / 16;            // k-steps that hold data
    static constexpr int AUGC = AUG_IN_PAD ? 8 : D;      // first extra column
    static constexpr int DT = (D + 31) / 32;
    static constexpr int DP = DT * 32;
    // The operand scaled by scale*log2(e) is rounded to 16 bits; for small head dims, where
    // the matrix core has k-steps to spare, its rounding residue is carried as well, which
    // makes the scores exact to fp32 (and identical in the forward and both backward kernels).
    static constexpr bool RESID = D <= 16;
    // From head dim 16 on the extra columns have a k-step of their own (the last).  The operand
    // that a wave keeps for a whole row holds zeros in that step's upper half (lane group 1), so
    // the operand read per tile may hold any finite values there: both lane groups read the same
    // extra columns, and no lane is cleared or masked per tile.
    static __device__ __forceinline__ constexpr bool aug_step(int ks) { return !AUG_IN_PAD && ks == KS - 1; }
};

template <typename T>
__device__ __forceinline__ typename Mfma<T>::v8 scaled8(typename Mfma<T>::v8 raw, float c) {
    typename Mfma<T>::v8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = (T)((float)raw[i] * c);
    return r;
}

// 8 operand columns [a0 a1 a2 b0 b1 b2 0 0] from two packed (hi, mid, lo, 0) triples.
template <typename T>
__device__ __forceinline__ typename Mfma<T>::v8 aug8(uint2 a, uint2 b) {
    typename Mfma<T>::v4 va = __builtin_bit_cast(typename Mfma<T>::v4, a);
    typename Mfma<T>::v4 vb = __builtin_bit_cast(typename Mfma<T>::v4, b);
    typename Mfma<T>::v8 r;
    r[0] = va[0]; r[1] = va[1]; r[2] = va[2];
    r[3] = vb[0]; r[4] = vb[1]; r[5] = vb[2];
    r[6] = (T)0.0f; r[7] = (T)0.0f;
    return r;
}

template <typename T>
__device__ __forceinline__ uint2 ones3() {
    typename Mfma<T>::v4 v;
    v[0] = v[1] = v[2] = (T)1.0f;
    v[3] = (T)0.0f;
    return __builtin_bit_cast(uint2, v);
}

// Raises a kernel's dynamic-LDS limit once per device (the attribute belongs to the device's
// copy of the kernel) and reports that device's CU count.  `done` is the caller's per-kernel
// state, one slot per device ordinal.  Host threads may make a kernel's first call on a device
// at the same time: the slot is published with release / acquire ordering after the attribute
// is set, and a thread that loses the race sets the same attribute to the same value again.
constexpr int kMaxDevices = 64;
struct PerDevice {
    std::atomic<int> cus[kMaxDevices];   // 0: not set up yet on that device
};
static inline int ensure_dynamic_lds(const void *kern, int bytes, PerDevice &done, int *cus) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return EVO_EHIP - (int)hipGetLastError();
    if (dev < 0 || dev >= kMaxDevices) return EVO_EUNSUPPORTED;
    int n = done.cus[dev].load(std::memory_order_acquire);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        const hipError_t err = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (err != hipSuccess) return EVO_EHIP - (int)err;
        done.cus[dev].store(n, std::memory_order_release);
    }
    if (cus) *cus = n;
    return EVO_OK;
}

static inline int hip_rc() {
    hipError_t err = hipGetLastError();
    return err == hipSuccess ? EVO_OK : EVO_EHIP - (int)err;
}

// The dBias partials that the dQ kernel left (one per chunk of its own) summed in chunk order and cast to the dBias
// dtype, a slice per workgroup, by the dK/dV kernel on its way in: no launch of its own for 16 bytes read per
// thread and chunk.  Needs B * H * N * N a multiple of 4 and a 16-byte aligned dBias (the caller checks).
template <int NTH>
__device__ __forceinline__ void sum_dbias_partials(const EvoAttnParams &p, const Extra &e, int tid) {
    const int64_t n = (int64_t)p.B * p.H * p.N * p.N;
    for (int64_t i = ((int64_t)blockIdx.x * NTH + tid) * 4; i < n; i += (int64_t)gridDim.x * NTH * 4) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int c0 = 0; c0 < e.dbias_chunks; c0 += 4) {
            f32x4 v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)   // four loads in flight; chunks past the last repeat it and are not added
                v[j] = *reinterpret_cast<const f32x4 *>(e.dbias_part + (int64_t)min(c0 + j, e.dbias_chunks - 1) * n + i);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (c0 + j < e.dbias_chunks) acc += v[j];
        }
        if (p.dbias_dtype == EVO_F32) {
            *reinterpret_cast<f32x4 *>((float *)p.dbias + i) = acc;
        } else if (p.dbias_dtype == EVO_BF16) {
            store4<bf16_t>((bf16_t *)p.dbias + i, acc[0], acc[1], acc[2], acc[3]);
        } else {
            store4<f16_t>((f16_t *)p.dbias + i, acc[0], acc[1], acc[2], acc[3]);
        }
    }
}

}  // namespace evo
