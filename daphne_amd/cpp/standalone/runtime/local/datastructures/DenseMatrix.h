// Stand-in for DAPHNE's src/runtime/local/datastructures/DenseMatrix.h (DenseMatrix): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>
