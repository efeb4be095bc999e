// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_BINARYOP_PARAMS_H
#define SNN_FWD_BINARYOP_PARAMS_H
#include "portdnn/hip/binaryop.h"
#endif
