// portDNN include path kept for source compatibility.
#ifndef SNN_FWD_BACKEND_HIP_BACKEND_H
#define SNN_FWD_BACKEND_HIP_BACKEND_H
#include "portdnn/hip/backend.h"
#endif
