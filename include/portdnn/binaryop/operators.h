// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_BINARYOP_OPERATORS_H
#define SNN_FWD_BINARYOP_OPERATORS_H
#include "portdnn/hip/binaryop.h"
#endif
