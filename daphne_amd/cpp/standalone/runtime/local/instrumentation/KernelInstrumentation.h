// Stand-in for DAPHNE's src/runtime/local/instrumentation/KernelInstrumentation.h (preKernelInstrumentation, postKernelInstrumentation): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
