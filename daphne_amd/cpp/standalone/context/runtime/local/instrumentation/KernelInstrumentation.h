// Stand-in for DAPHNE's src/runtime/local/instrumentation/KernelInstrumentation.h (preKernelInstrumentation, postKernelInstrumentation): see StandaloneContext.h.
#pragma once
#include <StandaloneContext.h>
