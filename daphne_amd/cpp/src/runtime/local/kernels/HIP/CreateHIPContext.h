// createHIPContext: the kernel the compiled program calls once at start-up when HIP is switched on
// (the counterpart of CUDA::createCUDAContext, src/runtime/local/kernels/CUDA/CreateCUDAContext.cpp:5-10,
// inserted by compiler/lowering/InsertDaphneContextPass.cpp:59-63). One context, device 0.
#pragma once

#include <runtime/local/context/DaphneContext.h>
#include <runtime/local/context/HIPContext.h>

namespace HIP {
inline void createHIPContext(DCTX(ctx)) { ctx->hip_contexts.emplace_back(HIPContext::createHipContext(0)); }
} // namespace HIP
