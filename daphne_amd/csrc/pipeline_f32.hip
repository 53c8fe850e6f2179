// Fused vectorized pipeline, float instantiation. See pipeline_impl.h for the design.
#include "pipeline_impl.h"

extern "C" dh_status dh_vectorized_pipeline_f32(dh_ctx *ctx, const dh_pipe_instr *program, int num_instr,
                                                const dh_pipe_io_f32 *io, size_t rows, size_t cols) {
    return dh_pipe::run<float, dh_pipe_io_f32>(ctx, program, num_instr, io, rows, cols);
}
