// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_HELPERS_RATIO_H
#define SNN_FWD_HELPERS_RATIO_H
#include "portdnn/hip/core.h"
#endif
