// Stand-in for DAPHNE's src/util/ErrorHandler.h (ErrorHandler, KernelDispatchMapping): see StandaloneContext.h.
#pragma once
#include <StandaloneContext.h>
