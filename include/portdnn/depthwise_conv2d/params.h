// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_DEPTHWISE_CONV2D_PARAMS_H
#define SNN_FWD_DEPTHWISE_CONV2D_PARAMS_H
#include "portdnn/hip/depthwise_conv2d.h"
#endif
