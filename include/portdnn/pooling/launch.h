// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_POOLING_LAUNCH_H
#define SNN_FWD_POOLING_LAUNCH_H
#include "portdnn/hip/pooling.h"
#endif
