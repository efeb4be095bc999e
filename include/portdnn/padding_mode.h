// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_PADDING_MODE_H
#define SNN_FWD_PADDING_MODE_H
#include "portdnn/hip/core.h"
#endif
