// Stand-in for DAPHNE's src/runtime/local/datastructures/DenseMatrix.h (DenseMatrix): see StandaloneData.h.
#pragma once
#include <StandaloneData.h>
