// Host-side launchers of the kernel families; each enqueues on `st` and returns EVO_OK or
// EVO_EHIP - hipError_t.
#pragma once

#include "common.h"

namespace evo {

int launch_generic_fwd(const EvoAttnParams &p, hipStream_t st);
int launch_generic_bwd(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_delta_generic(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_dmask_reduce(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_dbias_reduce(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_gate_bwd(const EvoAttnParams &p, void *dout_ungated, float *delta, hipStream_t st);  // dO, dgate and delta from the gradient of the gated output
int launch_mask_shift(const EvoAttnParams &p, const Extra &e, hipStream_t st);

int launch_prep(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_mfma_fwd(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_mfma_fwdr(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int mfma_fwdr_max_n(int D);  // largest N the chunk-of-rows forward takes, 0 for a head dim it is not built for
int launch_mfma_dq(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_mfma_dqr(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_mfma_kvr(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int mfma_kvr_max_n(int D);  // largest N the chunk-of-rows dK/dV kernel takes (it takes N > 128 only), 0 where it is not built
// whether the dQ kernel over a chunk of rows, where it serves such rows, also does the gate's backward pass on the
// rows it stages (its form of one stage of up to 256 keys with two query tiles, at head dim 32)
inline bool mfma_dqr_gate_ok(int D, int N) { return D == 32 && N <= 256; }
int mfma_dqr_qrows(int D, int N);  // query rows per workgroup of the double-buffered dQ kernel (64 or 32), 0 where it is not built for such rows
int launch_mfma_dkdv(const EvoAttnParams &p, const Extra &e, hipStream_t st);
int launch_mfma_dqw(const EvoAttnParams &p, const Extra &e, hipStream_t st);  // dQ where no dBias is asked for
int launch_mfma_dbias(const EvoAttnParams &p, const Extra &e, hipStream_t st);  // dBias partials alone (reads delta)

}  // namespace evo
