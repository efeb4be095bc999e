// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_POINTWISE_LAUNCH_H
#define SNN_FWD_POINTWISE_LAUNCH_H
#include "portdnn/hip/pointwise.h"
#endif
