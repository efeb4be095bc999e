// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_STATUS_H
#define SNN_FWD_STATUS_H
#include "portdnn/hip/core.h"
#endif
