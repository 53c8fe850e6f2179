// Stand-in for DAPHNE's src/runtime/local/datagen/GenGivenVals.h (genGivenVals): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
