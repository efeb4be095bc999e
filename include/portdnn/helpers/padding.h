// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_HELPERS_PADDING_H
#define SNN_FWD_HELPERS_PADDING_H
#include "portdnn/hip/core.h"
#endif
