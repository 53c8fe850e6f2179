// The whole HIP kernel layer in one include: every kernel header of src/runtime/local/kernels/HIP, the device
// context, the allocation descriptor and the vectorized-pipeline task. Include paths needed:
//   <this directory>/src          the files that go into DAPHNE's src/ tree (same relative paths)
//   <this directory>/standalone/context, <this directory>/standalone/data
//                                 stand-ins for DAPHNE's own headers; leave out when building inside DAPHNE
//   <repository>/include          daphne_hip.h, the C ABI of libdaphne_hip.so
#pragma once

#include <runtime/local/context/HIPContext.h>
#include <runtime/local/datastructures/AllocationDescriptorHIP.h>
#include <runtime/local/kernels/HIP/Activation.h>
#include <runtime/local/kernels/HIP/Affine.h>
#include <runtime/local/kernels/HIP/AggAll.h>
#include <runtime/local/kernels/HIP/AggCol.h>
#include <runtime/local/kernels/HIP/AggRow.h>
#include <runtime/local/kernels/HIP/BatchNorm.h>
#include <runtime/local/kernels/HIP/BatchNorm2DBackward.h>
#include <runtime/local/kernels/HIP/BatchNorm2DTrainForward.h>
#include <runtime/local/kernels/HIP/BiasAdd.h>
#include <runtime/local/kernels/HIP/ColBind.h>
#include <runtime/local/kernels/HIP/Conv2DBackwardData.h>
#include <runtime/local/kernels/HIP/Conv2DBackwardFilter.h>
#include <runtime/local/kernels/HIP/Convolution.h>
#include <runtime/local/kernels/HIP/CreateHIPContext.h>
#include <runtime/local/kernels/HIP/EwBinaryMat.h>
#include <runtime/local/kernels/HIP/EwBinaryObjSca.h>
#include <runtime/local/kernels/HIP/EwUnaryMat.h>
#include <runtime/local/kernels/HIP/ExtractCol.h>
#include <runtime/local/kernels/HIP/Fill.h>
#include <runtime/local/kernels/HIP/FusedOperators.h>
#include <runtime/local/kernels/HIP/FusedPipeline.h>
#include <runtime/local/kernels/HIP/Gemv.h>
#include <runtime/local/kernels/HIP/MatMul.h>
#include <runtime/local/kernels/HIP/OperatorChainMatcher.h>
#include <runtime/local/kernels/HIP/PipelineProgramBuilder.h>
#include <runtime/local/kernels/HIP/Pooling.h>
#include <runtime/local/kernels/HIP/PoolingBackward.h>
#include <runtime/local/kernels/HIP/Softmax.h>
#include <runtime/local/kernels/HIP/Solve.h>
#include <runtime/local/kernels/HIP/Syrk.h>
#include <runtime/local/kernels/HIP/Transpose.h>
#include <runtime/local/kernels/HIP/VectorizedPipeline.h>
#include <runtime/local/vectorized/TasksHIP.h>
