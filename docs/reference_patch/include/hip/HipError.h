// include/hip/HipError.h -- status check for calls into libpixienn_hip.so, the counterpart of
// PX_CUDA_CHECK_ERR / PX_CHECK_CUDNN (include/CudaError.h, include/Cudnn.h of the engine).
#pragma once

#include "pixienn_hip.h"

#define PX_HIP_CHECK(call)                                                              \
    do {                                                                                \
        const int px_hip_status_ = (call);                                              \
        if (px_hip_status_ != PXH_OK)                                                   \
            PX_ERROR_THROW("%s (status %d)", pxh_last_error(), px_hip_status_);         \
    } while (0)
