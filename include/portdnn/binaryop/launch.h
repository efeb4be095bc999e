// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_BINARYOP_LAUNCH_H
#define SNN_FWD_BINARYOP_LAUNCH_H
#include "portdnn/hip/binaryop.h"
#endif
