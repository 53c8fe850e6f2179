// Stand-in for the two enumerations of DAPHNE's src/runtime/local/vectorized/LoadPartitioningDefs.h:19-21 that a
// CPU worker's constructor takes.
#pragma once

enum class QueueTypeOption { CENTRALIZED, PERGROUP, PERCPU };
enum class VictimSelectionLogic { SEQ, SEQPRI, RANDOM, RANDOMPRI };
