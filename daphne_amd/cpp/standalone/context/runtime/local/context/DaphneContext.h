// Stand-in for DAPHNE's src/runtime/local/context/DaphneContext.h (IContext, DaphneContext, DCTX): see StandaloneContext.h.
#pragma once
#include <StandaloneContext.h>
