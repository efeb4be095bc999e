// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_FILTER_FORMAT_H
#define SNN_FWD_FILTER_FORMAT_H
#include "portdnn/hip/core.h"
#endif
