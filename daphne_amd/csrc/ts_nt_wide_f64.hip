// X t(C) in double with all eight chunks of a 64-column row in one step: the one instantiation of the streaming kernel
// that is compiled by itself, with the accumulators of the matrix instructions in ordinary vector registers
// (see ts_nt_launch_wide_f64 in ts_impl.h).
#include "ts_impl.h"

namespace dh_gemm {
dh_status ts_nt_launch_wide_f64(dh_ctx *ctx, const TsNtArgs &g, size_t lds) {
    return ts_nt_launch_cpg<double, 1, false, 8>(ctx, g, lds);
}
} // namespace dh_gemm
