// Instantiations of the walk kernels (fla_chunk_walk.h): both storage types, padded head dims 32, 64 and 128
// (128: backward is one reverse walk when forward handed its states over; otherwise, and with a feature map or
// the normaliser, dQ is a forward-direction walk and dK, dV a kernel of their own).
#include "fla_dispatch.h"

namespace fla {

#define FLA_WALK_DISPATCH(fn, ...)                                                       \
    if (dtype == 0) return D == 32 ? fn<__bf16, 32>(__VA_ARGS__) : fn<__bf16, 64>(__VA_ARGS__); \
    return D == 32 ? fn<_Float16, 32>(__VA_ARGS__) : fn<_Float16, 64>(__VA_ARGS__)

hipError_t walk_bwd(int dtype, int D, const WalkParams &p, hipStream_t stream) {
    if (D == 128) return hipErrorNotSupported;
    FLA_WALK_DISPATCH(launch_walk_bwd, p, stream);
}
#define FLA_WALK_DISPATCH3(fn, ...)                                                                 \
    if (D == 128) return dtype == 0 ? fn<__bf16, 128>(__VA_ARGS__) : fn<_Float16, 128>(__VA_ARGS__); \
    FLA_WALK_DISPATCH(fn, __VA_ARGS__)

hipError_t walk_dkdv(int dtype, int D, const WalkParams &p, hipStream_t stream) {
    if (D != 128) return hipErrorNotSupported;
    return dtype == 0 ? launch_walk_dkdv<__bf16, 128>(p, stream) : launch_walk_dkdv<_Float16, 128>(p, stream);
}
hipError_t walk_bwd_rev(int dtype, int D, const WalkParams &p, hipStream_t stream) {
    if (D != 128) return hipErrorNotSupported;
    return dtype == 0 ? launch_walk_bwd_rev<__bf16, 128>(p, stream) : launch_walk_bwd_rev<_Float16, 128>(p, stream);
}
hipError_t walk_totals(int dtype, int D, const WalkTotalsParams &p, hipStream_t stream) {
    FLA_WALK_DISPATCH3(launch_walk_totals, p, stream);
}
hipError_t walk_fwd(int dtype, int D, const WalkParams &p, hipStream_t stream) {
    FLA_WALK_DISPATCH3(launch_walk_fwd, p, stream);
}
hipError_t walk_fwd_wide(int dtype, const WalkParams &p, hipStream_t stream) {
    return dtype == 0 ? launch_walk_fwd_wide<__bf16>(p, stream) : launch_walk_fwd_wide<_Float16>(p, stream);
}
hipError_t walk_bwd_rev_wide(int dtype, const WalkParams &p, hipStream_t stream) {
    return dtype == 0 ? launch_walk_bwd_rev_wide<__bf16>(p, stream) : launch_walk_bwd_rev_wide<_Float16>(p, stream);
}
hipError_t walk_vec_sums(int dtype, int D, const WalkVecParams &p, int64_t BH, hipStream_t stream) {
    FLA_WALK_DISPATCH3(launch_walk_vec_sums, p, BH, stream);
}
hipError_t walk_vec_scan(float *v, int64_t BH, int n_chunks, int D, int reverse, hipStream_t stream) {
    return launch_walk_vec_scan(v, BH, n_chunks, D, reverse, stream);
}
hipError_t walk_scan(const float *totals, float *entry, int64_t BH, int n_seg, int D, int cols, int reverse,
                     hipStream_t stream, const float *totals_b, float *entry_b) {
    return launch_walk_scan(totals, entry, BH, n_seg, D, cols, reverse, stream, totals_b, entry_b);
}

}  // namespace fla

#include "fla_trace_structs.h"  // (the trace build's descriptions of the parameter structs; empty otherwise)
