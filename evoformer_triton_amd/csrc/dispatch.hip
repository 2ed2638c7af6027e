// Routes the matrix-core launches to the translation unit compiled for the head dim.
#include "common.h"
#include "kernels.h"

namespace evo {

#define EVO_DECL(D)                                                                          \
    int launch_mfma_fwd_d##D(const EvoAttnParams &, const Extra &, hipStream_t);             \
    int launch_mfma_fwdr_d##D(const EvoAttnParams &, const Extra &, hipStream_t);            \
    int mfma_fwdr_max_n_d##D();                                                              \
    int launch_mfma_dq_d##D(const EvoAttnParams &, const Extra &, hipStream_t);              \
    int launch_mfma_dqr_d##D(const EvoAttnParams &, const Extra &, hipStream_t);             \
    int mfma_dqr_qrows_d##D(int);                                                            \
    int launch_mfma_kvr_d##D(const EvoAttnParams &, const Extra &, hipStream_t);             \
    int mfma_kvr_max_n_d##D();                                                               \
    int launch_mfma_dkdv_d##D(const EvoAttnParams &, const Extra &, hipStream_t);            \
    int launch_mfma_dqw_d##D(const EvoAttnParams &, const Extra &, hipStream_t);             \
    int launch_mfma_dbias_d##D(const EvoAttnParams &, const Extra &, hipStream_t);
EVO_DECL(8)
EVO_DECL(16)
EVO_DECL(32)
EVO_DECL(64)
#undef EVO_DECL
// head dim 128: the one-workgroup-per-problem kernels only
int launch_mfma_fwd_d128(const EvoAttnParams &, const Extra &, hipStream_t);
int launch_mfma_dq_d128(const EvoAttnParams &, const Extra &, hipStream_t);
int launch_mfma_dkdv_d128(const EvoAttnParams &, const Extra &, hipStream_t);
int launch_mfma_dqw_d128(const EvoAttnParams &, const Extra &, hipStream_t);
static int unbuilt(const EvoAttnParams &, const Extra &, hipStream_t) { return EVO_EUNSUPPORTED; }
#define launch_mfma_fwdr_d128 unbuilt
#define launch_mfma_dqr_d128 unbuilt
#define launch_mfma_kvr_d128 unbuilt
#define launch_mfma_dbias_d128 unbuilt

#define EVO_ROUTE(name)                                                       \
    int launch_mfma_##name(const EvoAttnParams &p, const Extra &e, hipStream_t st) { \
        switch (p.D) {                                                        \
            case 8: return launch_mfma_##name##_d8(p, e, st);                 \
            case 16: return launch_mfma_##name##_d16(p, e, st);               \
            case 32: return launch_mfma_##name##_d32(p, e, st);               \
            case 64: return launch_mfma_##name##_d64(p, e, st);               \
            case 128: return launch_mfma_##name##_d128(p, e, st);             \
        }                                                                     \
        return EVO_EUNSUPPORTED;                                              \
    }
EVO_ROUTE(fwd)
EVO_ROUTE(fwdr)
EVO_ROUTE(dq)
EVO_ROUTE(dqr)
EVO_ROUTE(kvr)
EVO_ROUTE(dkdv)
EVO_ROUTE(dqw)
EVO_ROUTE(dbias)
#undef EVO_ROUTE

int mfma_fwdr_max_n(int D) {
    switch (D) {
        case 8: return mfma_fwdr_max_n_d8();
        case 16: return mfma_fwdr_max_n_d16();
        case 32: return mfma_fwdr_max_n_d32();
        case 64: return mfma_fwdr_max_n_d64();
    }
    return 0;
}

int mfma_kvr_max_n(int D) {
    switch (D) {
        case 8: return mfma_kvr_max_n_d8();
        case 16: return mfma_kvr_max_n_d16();
        case 32: return mfma_kvr_max_n_d32();
        case 64: return mfma_kvr_max_n_d64();
    }
    return 0;
}

int mfma_dqr_qrows(int D, int N) {
    switch (D) {
        case 8: return mfma_dqr_qrows_d8(N);
        case 16: return mfma_dqr_qrows_d16(N);
        case 32: return mfma_dqr_qrows_d32(N);
        case 64: return mfma_dqr_qrows_d64(N);
    }
    return 0;
}

}  // namespace evo
