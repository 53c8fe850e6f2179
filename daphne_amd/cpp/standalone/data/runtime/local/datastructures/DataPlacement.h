// Stand-in for DAPHNE's src/runtime/local/datastructures/DataPlacement.h (DataPlacement): see StandaloneData.h.
#pragma once
#include <StandaloneData.h>
