// Stand-in for DAPHNE's src/runtime/local/datastructures/DataPlacement.h (DataPlacement): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
