// The mat-vec launch family of one weight-format engine (see mmvq_launch.h).
#include "mmvq_launch.h"

LK_DEFINE_ENGINE(q6k_short, mmvq::EngQ6KShort)
