// Stand-in for DAPHNE's src/runtime/local/datastructures/DataObjectFactory.h (DataObjectFactory): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
