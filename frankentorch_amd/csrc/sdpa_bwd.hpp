// Internal entry points of the fused fp32 SDPA backward (csrc/sdpa_bwd.hip), used by csrc/backward.hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace fth {

// True when the fused path covers the problem: d_k == d_v in {64, 128}, sequence lengths of at least 32, a positive scale. Operands are contiguous [num_bh, seq, d] and 16-byte aligned (the caller checks the pointers).
bool sdpa_backward_fused_applies(int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d_k, int64_t d_v, float scale);

// Sizes, in floats, of the two score-shaped workspace arrays of the fused path: `s` holds the raw scores, `d` holds dP
// and then dS. Both are cut into 32 x 32 tiles per (batch, head), edge tiles stored whole, and `d` has one spare tile row.
void sdpa_backward_fused_workspace(int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t *s_floats, int64_t *d_floats);

// Launch 1: raw scores Q.K^T into s_out and dP = dOut.V^T into dp_out (tiled; only the tiles a causal problem uses are
// written), the rows' log-sum-exp in log2 units and delta_i = sum_j P_ij dP_ij. `dout_bh_stride` is seq_q * d, or 0 for
// one shared plane.
int32_t sdpa_backward_stats_f32(const float *q, const float *k, const float *v, const float *dout, int64_t dout_bh_stride, int64_t num_bh,
                                int64_t seq_q, int64_t seq_k, int64_t d, float scale, int causal, float *s_out, float *dp_out,
                                float *lse_out, float *delta_out, hipStream_t st);

// Launch 2: dS = P (dP - delta) into the array that holds dP (`dpds`, a tile row apart), dK and dV. Under a causal mask a
// key block walks the query rows from the start of the `row_block`-row block that holds its first key (row_block a
// multiple of 128; 0: from row 0) and writes the tiles it sees something of, zeros where masked: all the dQ pass reads.
int32_t sdpa_backward_keys_f32(const float *q, const float *dout, int64_t dout_bh_stride, const float *s, const float *lse,
                               const float *delta, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d, float scale, int causal,
                               int64_t row_block, float *dpds, float *dk, float *dv, hipStream_t st);

// Launch 3: dQ = scale . dS . K from the (unscaled) dS of launch 2 (contiguous [num_bh, seq, d] operands).
int32_t sdpa_backward_dq_f32(const float *ds, const float *k, int64_t num_bh, int64_t seq_q, int64_t seq_k, int64_t d, float scale,
                             int causal, float *dq, hipStream_t st);

}  // namespace fth
