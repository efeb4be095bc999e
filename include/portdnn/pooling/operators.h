// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_POOLING_OPERATORS_H
#define SNN_FWD_POOLING_OPERATORS_H
#include "portdnn/hip/pooling.h"
#endif
