// Stand-in for DAPHNE's src/runtime/local/datastructures/Structure.h (Structure): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
