// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_POOLING_SIZES_H
#define SNN_FWD_POOLING_SIZES_H
#include "portdnn/hip/pooling.h"
#endif
