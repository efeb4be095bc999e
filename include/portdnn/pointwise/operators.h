// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_POINTWISE_OPERATORS_H
#define SNN_FWD_POINTWISE_OPERATORS_H
#include "portdnn/hip/pointwise.h"
#endif
