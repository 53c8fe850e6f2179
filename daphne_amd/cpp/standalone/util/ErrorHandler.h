// Stand-in for DAPHNE's src/util/ErrorHandler.h (ErrorHandler, KernelDispatchMapping): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
