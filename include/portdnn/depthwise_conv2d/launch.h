// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_DEPTHWISE_CONV2D_LAUNCH_H
#define SNN_FWD_DEPTHWISE_CONV2D_LAUNCH_H
#include "portdnn/hip/depthwise_conv2d.h"
#endif
