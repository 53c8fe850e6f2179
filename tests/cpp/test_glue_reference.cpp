// The placement and vectorized-pipeline tests of placement_and_tasks.h, compiled against the reference's own
// DenseMatrix / MetaDataObject / DataPlacement / Structure sources (with patches/0011-dense-matrix-device-views.patch
// applied to a copy) instead of the stand-in data structures, and linked with mock_daphne_hip.cpp, a host-memory
// implementation of the C ABI. It shows that the C++ kernel layer - HIPContext, AllocationDescriptorHIP, the
// HIP::*::apply headers, CompiledPipelineTaskHIP, HIP::VectorizedPipeline - is type- and semantics-correct on
// DAPHNE's real data objects: more than one share or batch gives the one-share result, views reach their own rows.
// Built and run by tests/test_reference_datastructures.py where the reference tree is present.
#include <runtime/local/context/HIPContext.h>
#include <runtime/local/datastructures/AllocationDescriptorHIP.h>
#include <runtime/local/kernels/HIP/AggAll.h>
#include <runtime/local/kernels/HIP/AggCol.h>
#include <runtime/local/kernels/HIP/AggRow.h>
#include <runtime/local/kernels/HIP/CreateHIPContext.h>
#include <runtime/local/kernels/HIP/EwBinaryMat.h>
#include <runtime/local/kernels/HIP/EwBinaryObjSca.h>
#include <runtime/local/kernels/HIP/EwUnaryMat.h>
#include <runtime/local/kernels/HIP/Fill.h>
#include <runtime/local/kernels/HIP/FusedPipeline.h>
#include <runtime/local/kernels/HIP/VectorizedPipeline.h>
#include <runtime/local/vectorized/TasksHIP.h>

#define DAPHNE_HIP_KERNELS_INCLUDED_PIECEWISE
#include "placement_and_tasks.h"

#include <cstdio>
#include <memory>

int main() {
    auto dctx = std::make_unique<DaphneContext>();
    HIP::createHIPContext(dctx.get());
    CHECK(dctx->useHIP());
    run_placement(dctx.get());
    run_pipeline_tasks<float>(dctx.get());
    run_pipeline_tasks<double>(dctx.get());
    run_hybrid_pipeline<float>(dctx.get());
    run_hybrid_pipeline<double>(dctx.get());
    std::printf("%s: %d checks, %d failed\n", g_fail ? "FAILED" : "PASSED", g_checks, g_fail);
    return g_fail ? 1 : 0;
}
