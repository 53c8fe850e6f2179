// Stand-in for DAPHNE's src/runtime/local/datastructures/Structure.h (Structure): see StandaloneData.h.
#pragma once
#include <StandaloneData.h>
