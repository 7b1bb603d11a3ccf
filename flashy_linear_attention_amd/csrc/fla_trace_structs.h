// Field-by-field description of the kernels' parameter structs for the launch recorder of the
// host-only trace build (fla_trace.h).  Included at the end of a translation unit, once every
// struct is defined; found by argument-dependent lookup from launch_kernel.
#pragma once

#if defined(FLA_TRACE_LAUNCHES)

#include "fla_chunk_state.h"
#include "fla_chunk_walk.h"
#include "fla_norm.h"
#include "fla_tri_kernel.h"
#include "fla_tri_pair.h"

namespace fla {

// FLA_FIELD(name) writes r.field(arg, "<prefix><name>", p.<name>)
#define FLA_FIELDS_BEGIN(Type)                                              \
    inline void trace_fields(trace::Record &r, int arg, const std::string &pre, const Type &p) {
#define FLA_FIELD(name) r.field(arg, (pre + #name).c_str(), p.name);
#define FLA_FIELDS_END }

FLA_FIELDS_BEGIN(TriParams)
FLA_FIELD(x) FLA_FIELD(y) FLA_FIELD(z) FLA_FIELD(out)
FLA_FIELD(xs_b) FLA_FIELD(xs_h) FLA_FIELD(xs_n) FLA_FIELD(ys_b) FLA_FIELD(ys_h) FLA_FIELD(ys_n)
FLA_FIELD(zs_b) FLA_FIELD(zs_h) FLA_FIELD(zs_n) FLA_FIELD(os_b) FLA_FIELD(os_h) FLA_FIELD(os_n)
FLA_FIELD(H) FLA_FIELD(N) FLA_FIELD(BH) FLA_FIELD(dc) FLA_FIELD(dout) FLA_FIELD(upper) FLA_FIELD(n_tiles)
FLA_FIELD(single) FLA_FIELD(vec_x) FLA_FIELD(vec_y) FLA_FIELD(vec_z) FLA_FIELD(vec_out) FLA_FIELD(state)
FLA_FIELD(state_transposed) FLA_FIELD(denom) FLA_FIELD(eps) FLA_FIELD(poly_on) FLA_FIELD(map_x) FLA_FIELD(map_out)
FLA_FIELD(xmap_out) FLA_FIELD(xo_b) FLA_FIELD(xo_h) FLA_FIELD(xo_n) FLA_FIELD(omap) FLA_FIELD(ms_b) FLA_FIELD(ms_h)
FLA_FIELD(ms_n)
FLA_FIELDS_END

FLA_FIELDS_BEGIN(TriPairParams)
FLA_FIELD(xa) FLA_FIELD(xb) FLA_FIELD(ya) FLA_FIELD(yb) FLA_FIELD(oa) FLA_FIELD(ob)
FLA_FIELD(xas_b) FLA_FIELD(xas_h) FLA_FIELD(xas_n) FLA_FIELD(xbs_b) FLA_FIELD(xbs_h) FLA_FIELD(xbs_n)
FLA_FIELD(yas_b) FLA_FIELD(yas_h) FLA_FIELD(yas_n) FLA_FIELD(ybs_b) FLA_FIELD(ybs_h) FLA_FIELD(ybs_n)
FLA_FIELD(oas_b) FLA_FIELD(oas_h) FLA_FIELD(oas_n) FLA_FIELD(obs_b) FLA_FIELD(obs_h) FLA_FIELD(obs_n)
FLA_FIELD(H) FLA_FIELD(N) FLA_FIELD(BH) FLA_FIELD(wa) FLA_FIELD(wb) FLA_FIELD(n_tiles) FLA_FIELD(single)
FLA_FIELDS_END

FLA_FIELDS_BEGIN(NormParams)
FLA_FIELD(q) FLA_FIELD(k) FLA_FIELD(a) FLA_FIELD(b) FLA_FIELD(out) FLA_FIELD(dq) FLA_FIELD(dk) FLA_FIELD(denom)
FLA_FIELD(dn) FLA_FIELD(ksum) FLA_FIELD(wsum)
FLA_FIELD(qs_b) FLA_FIELD(qs_h) FLA_FIELD(qs_n) FLA_FIELD(ks_b) FLA_FIELD(ks_h) FLA_FIELD(ks_n)
FLA_FIELD(as_b) FLA_FIELD(as_h) FLA_FIELD(as_n) FLA_FIELD(bs_b) FLA_FIELD(bs_h) FLA_FIELD(bs_n)
FLA_FIELD(os_b) FLA_FIELD(os_h) FLA_FIELD(os_n) FLA_FIELD(dqs_b) FLA_FIELD(dqs_h) FLA_FIELD(dqs_n)
FLA_FIELD(dks_b) FLA_FIELD(dks_h) FLA_FIELD(dks_n)
FLA_FIELD(H) FLA_FIELD(N) FLA_FIELD(BH) FLA_FIELD(dqk) FLA_FIELD(dv) FLA_FIELD(n_chunks)
FLA_FIELD(vec_q) FLA_FIELD(vec_k) FLA_FIELD(vec_a) FLA_FIELD(vec_b) FLA_FIELD(vec_out) FLA_FIELD(vec_dq)
FLA_FIELD(vec_dk) FLA_FIELD(eps) FLA_FIELD(fmap) FLA_FIELD(only_dk)
FLA_FIELDS_END

FLA_FIELDS_BEGIN(WalkParams)
FLA_FIELD(q) FLA_FIELD(k) FLA_FIELD(v) FLA_FIELD(go) FLA_FIELD(o) FLA_FIELD(dq) FLA_FIELD(dk) FLA_FIELD(dv)
FLA_FIELD(qs_b) FLA_FIELD(qs_h) FLA_FIELD(qs_n) FLA_FIELD(ks_b) FLA_FIELD(ks_h) FLA_FIELD(ks_n)
FLA_FIELD(vs_b) FLA_FIELD(vs_h) FLA_FIELD(vs_n) FLA_FIELD(gs_b) FLA_FIELD(gs_h) FLA_FIELD(gs_n)
FLA_FIELD(os_b) FLA_FIELD(os_h) FLA_FIELD(os_n) FLA_FIELD(dqs_b) FLA_FIELD(dqs_h) FLA_FIELD(dqs_n)
FLA_FIELD(dks_b) FLA_FIELD(dks_h) FLA_FIELD(dks_n) FLA_FIELD(dvs_b) FLA_FIELD(dvs_h) FLA_FIELD(dvs_n)
FLA_FIELD(H) FLA_FIELD(N) FLA_FIELD(BH) FLA_FIELD(wqk) FLA_FIELD(wv) FLA_FIELD(n_chunks) FLA_FIELD(seg_chunks)
FLA_FIELD(n_seg) FLA_FIELD(init) FLA_FIELD(init_transposed) FLA_FIELD(saved) FLA_FIELD(fmap) FLA_FIELD(qmap_out)
FLA_FIELD(qo_b) FLA_FIELD(qo_h) FLA_FIELD(qo_n) FLA_FIELD(slope_y) FLA_FIELD(sy_b) FLA_FIELD(sy_h) FLA_FIELD(sy_n)
FLA_FIELD(denom) FLA_FIELD(eps) FLA_FIELD(zc) FLA_FIELD(dn) FLA_FIELD(rc) FLA_FIELD(total_out) FLA_FIELD(xinit)
FLA_FIELD(xtotal) FLA_FIELD(accumulate)
    FLA_FIELD(wqk2) FLA_FIELD(init2) FLA_FIELD(total_out2) FLA_FIELD(xinit2) FLA_FIELD(xtotal2)
    FLA_FIELD(init_is_totals) FLA_FIELD(entry_out) FLA_FIELD(entry_out2)
FLA_FIELDS_END

FLA_FIELDS_BEGIN(WalkTotalsParams)
FLA_FIELD(y) FLA_FIELD(z) FLA_FIELD(ys_b) FLA_FIELD(ys_h) FLA_FIELD(ys_n) FLA_FIELD(zs_b) FLA_FIELD(zs_h)
FLA_FIELD(zs_n) FLA_FIELD(H) FLA_FIELD(N) FLA_FIELD(BH) FLA_FIELD(dy) FLA_FIELD(dz) FLA_FIELD(n_chunks)
FLA_FIELD(seg_chunks) FLA_FIELD(n_seg) FLA_FIELD(seg_lo) FLA_FIELD(seg_hi) FLA_FIELD(totals) FLA_FIELD(direct)
FLA_FIELD(map_y) FLA_FIELD(ymap_out) FLA_FIELD(yo_b) FLA_FIELD(yo_h) FLA_FIELD(yo_n) FLA_FIELD(y2) FLA_FIELD(dy2)
FLA_FIELD(totals2)
FLA_FIELDS_END

FLA_FIELDS_BEGIN(WalkVecParams)
FLA_FIELD(y) FLA_FIELD(ys_b) FLA_FIELD(ys_h) FLA_FIELD(ys_n) FLA_FIELD(w) FLA_FIELD(H) FLA_FIELD(N) FLA_FIELD(width)
FLA_FIELD(n_chunks) FLA_FIELD(out)
FLA_FIELDS_END

FLA_FIELDS_BEGIN(ChunkStateParams)
FLA_FIELD(y) FLA_FIELD(z) FLA_FIELD(w) FLA_FIELD(ys_b) FLA_FIELD(ys_h) FLA_FIELD(ys_n) FLA_FIELD(zs_b) FLA_FIELD(zs_h)
FLA_FIELD(zs_n) FLA_FIELD(H) FLA_FIELD(N) FLA_FIELD(BH) FLA_FIELD(dc) FLA_FIELD(dout) FLA_FIELD(n_chunks)
FLA_FIELD(map_y) FLA_FIELD(ymap_out) FLA_FIELD(yo_b) FLA_FIELD(yo_h) FLA_FIELD(yo_n)
FLA_FIELDS_END

#undef FLA_FIELDS_BEGIN
#undef FLA_FIELD
#undef FLA_FIELDS_END

inline void trace_describe(trace::Record &r, int arg, const TriParams &p) { trace_fields(r, arg, "", p); }
inline void trace_describe(trace::Record &r, int arg, const TriPairParams &p) { trace_fields(r, arg, "", p); }
inline void trace_describe(trace::Record &r, int arg, const NormParams &p) { trace_fields(r, arg, "", p); }
inline void trace_describe(trace::Record &r, int arg, const WalkParams &p) { trace_fields(r, arg, "", p); }
inline void trace_describe(trace::Record &r, int arg, const WalkTotalsParams &p) { trace_fields(r, arg, "", p); }
inline void trace_describe(trace::Record &r, int arg, const WalkVecParams &p) { trace_fields(r, arg, "", p); }
inline void trace_describe(trace::Record &r, int arg, const ChunkStateParams &p) { trace_fields(r, arg, "", p); }
inline void trace_describe(trace::Record &r, int arg, const TriBatch &b) {
    for (int i = 0; i < 3; ++i) trace_fields(r, arg, "p" + std::to_string(i) + ".", b.p[i]);
}

}  // namespace fla

#endif  // FLA_TRACE_LAUNCHES
