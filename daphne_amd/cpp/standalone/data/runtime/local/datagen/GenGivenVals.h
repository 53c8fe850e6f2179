// Stand-in for DAPHNE's src/runtime/local/datagen/GenGivenVals.h (genGivenVals): see StandaloneData.h.
#pragma once
#include <StandaloneData.h>
