// Instantiations of the fused dV + dK kernel (fla_tri_pair.h) at padded head dim 128, both storage
// types.  A translation unit of its own because it is compiled WITHOUT -amdgpu-mfma-vgpr-form: with
// that option the compiler's pass that rewrites accumulation-register copies fails on this kernel,
// and here the two sets of accumulators (128 registers that only MFMAs touch between the first
// tile and the epilogue) belong in accumulation registers anyway.
#include "fla_dispatch.h"
#include "fla_tri_fast.h"
#include "fla_tri_pair.h"

namespace fla {

hipError_t FLA_PAIR_NAME(0, 128)(const TriParams &a, const TriParams &b, hipStream_t stream) {
    return launch_tri_pair<__bf16, 128>(a, b, stream);
}
hipError_t FLA_PAIR_NAME(1, 128)(const TriParams &a, const TriParams &b, hipStream_t stream) {
    return launch_tri_pair<_Float16, 128>(a, b, stream);
}

}  // namespace fla

#include "fla_trace_structs.h"  // (the trace build's descriptions of the parameter structs; empty otherwise)
