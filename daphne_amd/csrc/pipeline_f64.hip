// Fused vectorized pipeline, double instantiation. See pipeline_impl.h for the design.
#include "pipeline_impl.h"

extern "C" dh_status dh_vectorized_pipeline_f64(dh_ctx *ctx, const dh_pipe_instr *program, int num_instr,
                                                const dh_pipe_io_f64 *io, size_t rows, size_t cols) {
    return dh_pipe::run<double, dh_pipe_io_f64>(ctx, program, num_instr, io, rows, cols);
}
