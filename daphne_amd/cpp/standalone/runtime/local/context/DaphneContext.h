// Stand-in for DAPHNE's src/runtime/local/context/DaphneContext.h (IContext, DaphneContext, DCTX): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
