// Stand-in for DAPHNE's src/runtime/local/datastructures/DataObjectFactory.h (DataObjectFactory): see StandaloneData.h.
#pragma once
#include <StandaloneData.h>
