// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_MATMUL_LAUNCH_H
#define SNN_FWD_MATMUL_LAUNCH_H
#include "portdnn/hip/matmul.h"
#endif
