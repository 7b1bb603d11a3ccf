// One kernel instantiation per compilation: build with
//   -DFLA_INST_DTYPE={0 bf16 | 1 f16} -DFLA_INST_DC=<32|64|128|256> -DFLA_INST_DO=<32|64|128|256>
#include "fla_dispatch.h"
#include "fla_tri_fast.h"
#include "fla_tri_pair.h"

#if !defined(FLA_INST_DTYPE) || !defined(FLA_INST_DC) || !defined(FLA_INST_DO)
#error "define FLA_INST_DTYPE, FLA_INST_DC and FLA_INST_DO"
#endif

namespace fla {

#if FLA_INST_DTYPE == 0
using InstT = __bf16;
#else
using InstT = _Float16;
#endif

hipError_t FLA_LAUNCH_NAME(FLA_INST_DTYPE, FLA_INST_DC, FLA_INST_DO)(const TriParams &p, hipStream_t stream) {
    // aligned operands take the LDS-DMA pipelined kernel; anything else (odd
    // widths, unaligned rows, slices beyond 1 GiB, tiles too big for three LDS
    // stages) takes the bounds-checked generic kernel
    if (FastConfig<FLA_INST_DC, FLA_INST_DO>::kSupported && fast_path_ok(p))
        return launch_tri_fast<InstT, FLA_INST_DC, FLA_INST_DO>(p, stream);
    if (p.map_x || p.omap) return hipErrorNotSupported;  // feature maps: fast path only
    return launch_tri<InstT, FLA_INST_DC, FLA_INST_DO>(p, stream);
}

hipError_t FLA_STATE_NAME(FLA_INST_DTYPE, FLA_INST_DC, FLA_INST_DO)(const ChunkStateParams &p, hipStream_t stream) {
    return launch_chunk_state<InstT, FLA_INST_DC, FLA_INST_DO>(p, stream);
}

#if FLA_INST_DC == FLA_INST_DO
hipError_t FLA_BATCH_NAME(FLA_INST_DTYPE, FLA_INST_DC)(const TriBatch &b, int count, hipStream_t stream) {
    if (!FastConfig<FLA_INST_DC, FLA_INST_DO>::kSupported) return hipErrorNotSupported;
    return launch_tri_fast_batch<InstT, FLA_INST_DC, FLA_INST_DO>(b, count, stream);
}

hipError_t FLA_CBATCH_NAME(FLA_INST_DTYPE, FLA_INST_DC)(const TriBatch &b, int count, hipStream_t stream) {
    return launch_tri_fast_chunked_batch<InstT, FLA_INST_DC, FLA_INST_DO>(b, count, stream);
}
#endif

#if FLA_INST_DC == FLA_INST_DO && FLA_INST_DC <= 64  // (128: fla_pair_inst.hip)
hipError_t FLA_PAIR_NAME(FLA_INST_DTYPE, FLA_INST_DC)(const TriParams &a, const TriParams &b, hipStream_t stream) {
    return launch_tri_pair<InstT, FLA_INST_DC>(a, b, stream);
}
#endif

#if FLA_INST_DTYPE == 0
// rows per chunk of the chunked evaluation = row tile of the fast kernel (0: no fast kernel)
#define FLA_CHUNK_ROWS_NAME_(dc, dout) fla_chunk_rows_c##dc##_o##dout
#define FLA_CHUNK_ROWS_NAME(dc, dout) FLA_CHUNK_ROWS_NAME_(dc, dout)
int FLA_CHUNK_ROWS_NAME(FLA_INST_DC, FLA_INST_DO)() {
    return FastConfig<FLA_INST_DC, FLA_INST_DO>::kSupported ? FastConfig<FLA_INST_DC, FLA_INST_DO>::BM : 0;
}
#endif

}  // namespace fla

#include "fla_trace_structs.h"  // (the trace build's descriptions of the parameter structs; empty otherwise)
