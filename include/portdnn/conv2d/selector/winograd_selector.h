// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_CONV2D_SELECTOR_WINOGRAD_SELECTOR_H
#define SNN_FWD_CONV2D_SELECTOR_WINOGRAD_SELECTOR_H
#include "portdnn/hip/conv2d.h"
#endif
