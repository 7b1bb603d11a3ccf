// Declarations shared by the per-instantiation translation units and the C ABI.
#pragma once

#include <hip/hip_runtime.h>

#include "fla_chunk_state.h"
#include "fla_chunk_walk.h"
#include "fla_tri_kernel.h"

// Padded (DC, DO) pairs for which a kernel is built.  Widths are padded to the
// next of 32/64/128/256, as the reference pads to the next power of two
// (flashlinear/kernels/linear_attn_kernels.py:316).
#define FLA_FOR_EACH_DIM_PAIR(X)                                                               \
    X(32, 32) X(32, 64) X(32, 128) X(32, 256) X(64, 32) X(64, 64) X(64, 128) X(64, 256)        \
    X(128, 32) X(128, 64) X(128, 128) X(128, 256) X(256, 32) X(256, 64) X(256, 128) X(256, 256)

#define FLA_LAUNCH_NAME_(t, dc, dout) fla_launch_tri_t##t##_c##dc##_o##dout
#define FLA_LAUNCH_NAME(t, dc, dout) FLA_LAUNCH_NAME_(t, dc, dout)
#define FLA_STATE_NAME_(t, dc, dout) fla_launch_state_t##t##_c##dc##_o##dout
#define FLA_STATE_NAME(t, dc, dout) FLA_STATE_NAME_(t, dc, dout)
#define FLA_BATCH_NAME_(t, d) fla_launch_batch_t##t##_d##d
#define FLA_BATCH_NAME(t, d) FLA_BATCH_NAME_(t, d)
#define FLA_CBATCH_NAME_(t, d) fla_launch_chunked_batch_t##t##_d##d
#define FLA_CBATCH_NAME(t, d) FLA_CBATCH_NAME_(t, d)
#define FLA_PAIR_NAME_(t, d) fla_launch_pair_t##t##_d##d
#define FLA_PAIR_NAME(t, d) FLA_PAIR_NAME_(t, d)

namespace fla {
#define FLA_DECLARE(dc, dout)                                                               \
    hipError_t FLA_LAUNCH_NAME(0, dc, dout)(const TriParams &p, hipStream_t stream);        \
    hipError_t FLA_LAUNCH_NAME(1, dc, dout)(const TriParams &p, hipStream_t stream);        \
    hipError_t FLA_STATE_NAME(0, dc, dout)(const ChunkStateParams &p, hipStream_t stream);  \
    hipError_t FLA_STATE_NAME(1, dc, dout)(const ChunkStateParams &p, hipStream_t stream);  \
    int fla_chunk_rows_c##dc##_o##dout();
FLA_FOR_EACH_DIM_PAIR(FLA_DECLARE)
#undef FLA_DECLARE
// several products of one square shape in a single launch (fast path only; hipErrorNotSupported otherwise)
#define FLA_DECLARE_BATCH(d)                                                                  \
    hipError_t FLA_BATCH_NAME(0, d)(const TriBatch &b, int count, hipStream_t stream);        \
    hipError_t FLA_BATCH_NAME(1, d)(const TriBatch &b, int count, hipStream_t stream);        \
    hipError_t FLA_CBATCH_NAME(0, d)(const TriBatch &b, int count, hipStream_t stream);       \
    hipError_t FLA_CBATCH_NAME(1, d)(const TriBatch &b, int count, hipStream_t stream);
FLA_DECLARE_BATCH(32) FLA_DECLARE_BATCH(64) FLA_DECLARE_BATCH(128) FLA_DECLARE_BATCH(256)
#undef FLA_DECLARE_BATCH
// two upper products that stream the same tiles (fla_tri_pair.h: the backward's dV and dK), padded head dims up to 128
#define FLA_DECLARE_PAIR(d)                                                                          \
    hipError_t FLA_PAIR_NAME(0, d)(const TriParams &a, const TriParams &b, hipStream_t stream);      \
    hipError_t FLA_PAIR_NAME(1, d)(const TriParams &a, const TriParams &b, hipStream_t stream);
FLA_DECLARE_PAIR(32) FLA_DECLARE_PAIR(64) FLA_DECLARE_PAIR(128)
#undef FLA_DECLARE_PAIR
// walk kernels (fla_chunk_walk.h), dtype 0 bf16 / 1 f16, padded head dim D = 32, 64 or 128
// (walk_bwd: 32 and 64; walk_dkdv, walk_bwd_rev: 128)
hipError_t walk_totals(int dtype, int D, const WalkTotalsParams &p, hipStream_t stream);
hipError_t walk_fwd(int dtype, int D, const WalkParams &p, hipStream_t stream);
hipError_t walk_fwd_wide(int dtype, const WalkParams &p, hipStream_t stream);  // (q, k of 129 .. 256 columns)
hipError_t walk_bwd_rev_wide(int dtype, const WalkParams &p, hipStream_t stream);  // (... and v of at most 64)
hipError_t walk_bwd_rev(int dtype, int D, const WalkParams &p, hipStream_t stream);
hipError_t walk_bwd(int dtype, int D, const WalkParams &p, hipStream_t stream);
hipError_t walk_dkdv(int dtype, int D, const WalkParams &p, hipStream_t stream);
hipError_t walk_vec_sums(int dtype, int D, const WalkVecParams &p, int64_t BH, hipStream_t stream);
hipError_t walk_vec_scan(float *v, int64_t BH, int n_chunks, int D, int reverse, hipStream_t stream);
hipError_t walk_scan(const float *totals, float *entry, int64_t BH, int n_seg, int D, int cols, int reverse,
                     hipStream_t stream, const float *totals_b = nullptr, float *entry_b = nullptr);
}  // namespace fla
